// Shared device helpers for the gfx950 kernels: element types, conversions,
// wavefront (64 lanes) and block reductions, and the host-side error record.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define HAL_WAVE 64

// ---- host-side error record -------------------------------------------------
// Every entry point returns 0 on success; otherwise it has written a message
// that hal_last_error() returns.
extern "C" const char* hal_last_error();
int hal_fail(const char* fmt, ...);

#define HAL_CHECK_HIP(expr)                                                      \
  do {                                                                           \
    hipError_t _e = (expr);                                                      \
    if (_e != hipSuccess)                                                        \
      return hal_fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),     \
                      __FILE__, __LINE__);                                       \
  } while (0)

#define HAL_REQUIRE(cond, ...)                                                   \
  do {                                                                           \
    if (!(cond)) return hal_fail(__VA_ARGS__);                                   \
  } while (0)

#define HAL_LAUNCH_CHECK() HAL_CHECK_HIP(hipGetLastError())

// ---- element types ------------------------------------------------------------
// dtype codes shared with the Python side
enum { HAL_F32 = 0, HAL_BF16 = 1 };

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v.bits) << 16);
}

// two floats to two bf16 in one word (first in the low half), round to nearest even,
// with the hardware's conversion
typedef __attribute__((ext_vector_type(2))) __bf16 hal_bf16x2;
typedef __attribute__((ext_vector_type(2))) float hal_f32x2;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const hal_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hal_bf16x2));
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((u >> 16) | 0x0040u);
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = (uint16_t)(u >> 16);
  }
  return r;
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// load element i of an array whose element type is given at run time
__device__ __forceinline__ float load_as_f32(const void* p, int dtype, size_t i) {
  return dtype == HAL_F32 ? ((const float*)p)[i] : bf16_to_f32(((const bf16_t*)p)[i]);
}

// ---- vectors of four elements as floats (16-byte or 8-byte accesses) ----------------
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 t = *(const float4*)p;
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&v)[4]) {
  const uint2 t = *(const uint2*)p;
  v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&v)[4]) {
  uint2 t;
  t.x = pack_bf16x2(v[0], v[1]);
  t.y = pack_bf16x2(v[2], v[3]);
  *(uint2*)p = t;
}
__device__ __forceinline__ void load4_any(const void* p, int dtype, size_t i, float (&v)[4]) {
  if (dtype == HAL_F32) load4((const float*)p + i, v);
  else load4((const bf16_t*)p + i, v);
}

// ---- reductions -----------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, HAL_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = HAL_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, HAL_WAVE));
  return v;
}

// Where element (slot, d) of one kv head's part of a page lies, counted in elements from
// that part's start.  Plain: keys [slot][D], values transposed [D][slot].  Tiled (pages of
// a multiple of 32 tokens, head sizes of a multiple of 32): per block of 32 slots the keys
// and the values lie in the order in which the matrix-core attention kernel's waves load
// them, one contiguous KB per MFMA operand:
//   keys   [block][tile t of 16 keys][32-dim step ks][dim quad][key c][8 dims],
//          slot r of the block is key c = (r/8)*4 + r%4 of tile t = (r%8)/4;
//   values [block][16-dim tile dt][8-key group][dim][8 keys].
__host__ __device__ __forceinline__ size_t kv_key_offset(bool tiled, int page_size, int D, int slot,
                                                         int d) {
  if (!tiled) return (size_t)slot * D + d;
  const int r = slot % 32, t = (r % 8) / 4, c = (r / 8) * 4 + r % 4;
  const int ks = d / 32, quad = (d % 32) / 8;
  return (size_t)(slot / 32) * 32 * D + (((t * (D / 32) + ks) * 64 + quad * 16 + c) * 8 + d % 8);
}
__host__ __device__ __forceinline__ size_t kv_value_offset(bool tiled, int page_size, int D,
                                                           int slot, int d) {
  if (!tiled) return (size_t)d * page_size + slot;
  const int r = slot % 32;
  return (size_t)(slot / 32) * 32 * D + (((d / 16) * 64 + (r / 8) * 16 + d % 16) * 8 + r % 8);
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` is shared memory for 16 floats.  Safe to call repeatedly with the
// same scratch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % HAL_WAVE, wave = threadIdx.x / HAL_WAVE;
  const int n_waves = (blockDim.x + HAL_WAVE - 1) / HAL_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % HAL_WAVE, wave = threadIdx.x / HAL_WAVE;
  const int n_waves = (blockDim.x + HAL_WAVE - 1) / HAL_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < n_waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// Device helpers shared by the serving kernel libraries (each library is one
// translation unit and includes this once).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace {

using bf16 = __hip_bfloat16;

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16* p) { return __bfloat162float(*p); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16* p, float v) { *p = __float2bfloat16(v); }
// value after one rounding to the storage type
template <typename T> __device__ __forceinline__ float rnd(float v);
template <> __device__ __forceinline__ float rnd<float>(float v) { return v; }
template <> __device__ __forceinline__ float rnd<bf16>(float v) {
  return __bfloat162float(__float2bfloat16(v));
}

__device__ __forceinline__ short f2bf_bits(float f) {
  union { float f; unsigned u; } c;
  c.f = f;
  return (short)((c.u + 0x7FFF + ((c.u >> 16) & 1)) >> 16);
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// eight neighbouring values (16-byte aligned for bf16, 32 for float) widened
// to float, and back with one rounding
__device__ __forceinline__ void load8(const float* p, float (&x)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
  x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float (&x)[8]) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  x[0] = __uint_as_float(w.x << 16); x[1] = __uint_as_float(w.x & 0xffff0000u);
  x[2] = __uint_as_float(w.y << 16); x[3] = __uint_as_float(w.y & 0xffff0000u);
  x[4] = __uint_as_float(w.z << 16); x[5] = __uint_as_float(w.z & 0xffff0000u);
  x[6] = __uint_as_float(w.w << 16); x[7] = __uint_as_float(w.w & 0xffff0000u);
}
__device__ __forceinline__ void store8(float* p, const float (&x)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float (&x)[8]) {
  uint4 w;
  w.x = (unsigned short)f2bf_bits(x[0]) | ((unsigned)(unsigned short)f2bf_bits(x[1]) << 16);
  w.y = (unsigned short)f2bf_bits(x[2]) | ((unsigned)(unsigned short)f2bf_bits(x[3]) << 16);
  w.z = (unsigned short)f2bf_bits(x[4]) | ((unsigned)(unsigned short)f2bf_bits(x[5]) << 16);
  w.w = (unsigned short)f2bf_bits(x[6]) | ((unsigned)(unsigned short)f2bf_bits(x[7]) << 16);
  *reinterpret_cast<uint4*>(p) = w;
}

constexpr int NT = 256;  // threads per block for the row kernels

// every thread gets the block total; scratch holds NT/64 floats
__device__ __forceinline__ float block_sum(float x, float* scratch) {
  x = wave_sum(x);
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = x;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += scratch[i];
  __syncthreads();
  return t;
}

inline int nblocks(int64_t n, int b) {
  int64_t g = (n + b - 1) / b;
  return (int)(g < 1 ? 1 : (g > 4096 ? 4096 : g));
}


}  // namespace

#define BY_DTYPE(dt, CALL)            \
  do {                                \
    if ((dt) == 0) {                  \
      using T = float;                \
      CALL;                           \
    } else {                          \
      using T = bf16;                 \
      CALL;                           \
    }                                 \
  } while (0)


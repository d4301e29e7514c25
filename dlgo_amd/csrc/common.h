// Shared by every kernel file: element types, conversions, wave reductions and
// the error convention (an exported function returns nullptr on success, else a
// message that names what was refused).  Everything here is written for gfx950:
// 64-lane waves, MFMA, 160 KB of LDS per CU.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define DLGO_DTYPE_F32 0
#define DLGO_DTYPE_BF16 1

#define WAVE 64

typedef uint16_t bf16_t;   // storage only; arithmetic is always float

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even (the hardware conversion of gfx950)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}

// One rotation of a pair (x0, x1) by the angle whose cosine and sine are c and s.  Written as a product and one fused
// multiply-add, so that every kernel that rotates gives the same bits whatever the compiler would otherwise contract.
__device__ __forceinline__ float rotated_lo(float x0, float x1, float c, float s) { return __builtin_fmaf(-x1, s, x0 * c); }
__device__ __forceinline__ float rotated_hi(float x0, float x1, float c, float s) { return __builtin_fmaf(x0, s, x1 * c); }

// A pointer that is the same in every lane of the wave, made so for an instruction that wants it in scalar registers.
// The halves are taken as unsigned: readfirstlane returns an int, which would be sign-extended into the upper half.
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (const void*)(uintptr_t)(((uint64_t)hi << 32) | (uint64_t)lo);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int code = DLGO_DTYPE_F32;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
  // two and four consecutive elements at once; p is aligned to what is stored
  __device__ static __forceinline__ void store2(float* p, float a, float b) { *(float2*)p = make_float2(a, b); }
  __device__ static __forceinline__ void store4(float* p, float a, float b, float c, float d) { *(float4*)p = make_float4(a, b, c, d); }
};
template <> struct Elem<bf16_t> {
  static constexpr int code = DLGO_DTYPE_BF16;
  __device__ static __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  __device__ static __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  __device__ static __forceinline__ uint32_t pair(float a, float b) { return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16); }
  __device__ static __forceinline__ void store2(bf16_t* p, float a, float b) { *(uint32_t*)p = pair(a, b); }
  __device__ static __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) { *(uint2*)p = make_uint2(pair(a, b), pair(c, d)); }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of NW waves; every thread gets the result.  `red` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if (NW == 1) return v;
  const int w = threadIdx.x / WAVE;
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += red[i];
  return t;
}

static thread_local char dlgo_errbuf[512];
#define DLGO_FAIL(...)                                        \
  do {                                                        \
    snprintf(dlgo_errbuf, sizeof(dlgo_errbuf), __VA_ARGS__);  \
    return dlgo_errbuf;                                       \
  } while (0)
#define DLGO_REQUIRE(cond, ...) \
  do {                          \
    if (!(cond)) DLGO_FAIL(__VA_ARGS__); \
  } while (0)
#define DLGO_LAUNCH_CHECK(what)                                             \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) DLGO_FAIL("%s: launch failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

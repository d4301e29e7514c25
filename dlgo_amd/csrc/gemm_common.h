// Shared by the two files of matrix products: the epilogues.
//   store in the run dtype; add into the float32 residual stream; SwiGLU of interleaved gate/up rows
//   (out[t, f] = silu(y[2f]) * y[2f+1], computerex/dlgo ops/activation.go:8-19,36-38); store float32 (logits).
#pragma once
#include "common.h"

// One library per element type: -DDLGO_ELEM=0 (float32) or 1 (bfloat16), so that a model compiles what it runs in.
#ifndef DLGO_ELEM
#error "compile with -DDLGO_ELEM=0 (float32) or 1 (bfloat16)"
#endif
#if DLGO_ELEM == DLGO_DTYPE_F32
typedef float elem_t;
#elif DLGO_ELEM == DLGO_DTYPE_BF16
typedef bf16_t elem_t;
#else
#error "DLGO_ELEM must be 0 or 1"
#endif

// The float32 build computes in true float32 from here to the end of the file that includes this: no reduced-precision
// matrix instruction, no hardware approximation and no bfloat16 type can be named in it (exact_begin.h).
#if DLGO_ELEM == DLGO_DTYPE_F32
#define DLGO_EXACT_NO_BF16 1
#include "exact_begin.h"
#endif

enum { EPI_STORE = 0, EPI_ACCUM_F32 = 1, EPI_SWIGLU = 2, EPI_STORE_F32 = 3 };

// silu(z) = z / (1 + e^-z).  For a float32 result: the library's exponential and a true division.  For a bfloat16
// result: the hardware's exp2 and reciprocal, each good to about one unit in the last place of float32, which is 2^-15
// of what bfloat16 keeps; a quarter of the instructions, which a prompt's gate/up product feels.
template <typename T> __device__ __forceinline__ float silu_f(float z);
template <> __device__ __forceinline__ float silu_f<float>(float z) { return z / (1.0f + expf(-z)); }
#if DLGO_ELEM == DLGO_DTYPE_BF16
template <> __device__ __forceinline__ float silu_f<bf16_t>(float z) {
  return z * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z * -1.44269504088896341f));
}
#endif

// Four consecutive outputs n..n+3 of token t.
template <typename T, int EPI>
__device__ __forceinline__ void epilogue4(void* __restrict__ Y, int ldy, int N, int t, int n, float v0, float v1, float v2,
                                          float v3) {
  if (n >= N) return;
  const bool full = n + 3 < N;
  if (EPI == EPI_STORE) {
    T* y = (T*)Y + (size_t)t * ldy + n;
    if (full && (ldy & 3) == 0 && ((uintptr_t)y & (4 * sizeof(T) - 1)) == 0) {
      Elem<T>::store4(y, v0, v1, v2, v3);
    } else {
      const float v[4] = {v0, v1, v2, v3};
      for (int r = 0; r < 4 && n + r < N; ++r) Elem<T>::store(y + r, v[r]);
    }
  } else if (EPI == EPI_ACCUM_F32 || EPI == EPI_STORE_F32) {
    float* y = (float*)Y + (size_t)t * ldy + n;
    if (full && (ldy & 3) == 0 && ((uintptr_t)y & 15) == 0) {
      float4 o = make_float4(v0, v1, v2, v3);
      if (EPI == EPI_ACCUM_F32) {
        const float4 old = *(float4*)y;
        o.x += old.x;
        o.y += old.y;
        o.z += old.z;
        o.w += old.w;
      }
      *(float4*)y = o;
    } else {
      const float v[4] = {v0, v1, v2, v3};
      for (int r = 0; r < 4 && n + r < N; ++r) y[r] = (EPI == EPI_ACCUM_F32 ? y[r] : 0.f) + v[r];
    }
  } else {   // EPI_SWIGLU: rows (n, n+1) and (n+2, n+3) are (gate, up) pairs; N is even
    T* y = (T*)Y + (size_t)t * ldy + (n >> 1);
    if (n + 3 < N && (ldy & 1) == 0 && ((uintptr_t)y & (2 * sizeof(T) - 1)) == 0) {     // both halves at once
      Elem<T>::store2(y, silu_f<T>(v0) * v1, silu_f<T>(v2) * v3);
    } else {
      Elem<T>::store(y, silu_f<T>(v0) * v1);
      if (n + 3 < N) Elem<T>::store(y + 1, silu_f<T>(v2) * v3);
    }
  }
}


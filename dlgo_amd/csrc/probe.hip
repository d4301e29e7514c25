// Measurement aids, not part of any step: what the chip does when nothing stands in the way.
//   mfma_only_kernel: every wave issues 32x32x16 bfloat16 MFMAs on registers and nothing else, to see the rate the
//   matrix units sustain at the clock the chip settles at (the published peak assumes the boost clock).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16_t;

__global__ __launch_bounds__(256) void mfma_only_kernel(float* __restrict__ out, int iters) {
  probe_f32x16_t acc[4];
  probe_bf16x8_t a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = (__bf16)(0.001f * (float)(threadIdx.x + e));
    b[e] = (__bf16)(0.002f * (float)(threadIdx.x % 7 + e));
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// out: blocks * 256 floats.  Each of the blocks' four waves issues iters * 16 MFMAs of 32x32x16 (32768 flop each).
extern "C" const char* dlgo_probe_mfma(float* out, int blocks, int iters, hipStream_t stream) {
  DLGO_REQUIRE(out && blocks > 0 && iters > 0, "probe: bad arguments");
  hipLaunchKernelGGL(mfma_only_kernel, dim3(blocks), dim3(256), 0, stream, out, iters);
  DLGO_LAUNCH_CHECK("probe_mfma");
  return nullptr;
}

// RMSNorm over rows of the float32 residual stream, written in the run dtype:
//   out[i] = x[i] * (1 / sqrt(sum(x^2)/d + eps)) * w[i]
// as computerex/dlgo's ops/norm.go:10-32 and gpu/shaders/rmsnorm.comp:19-44 (one
// workgroup per vector, tree reduction).  The sum is accumulated in float32 in a
// fixed order that depends on d only, so a row's result does not depend on the
// batch it came in.  An optional row index gathers rows first (the final norm
// runs on the rows whose logits are wanted only, models/llm/forward_batch.go:222-229).
#include "common.h"
// everything here is float32 arithmetic whatever the storage type: no approximation can be named (exact_begin.h)
#include "exact_begin.h"

// A thread keeps its part of the row (up to HOLD pieces of four floats) in registers between the sum and the write,
// so that a row is read once; longer rows are read a second time.
template <typename TO, int NW>
__global__ __launch_bounds__(NW * WAVE) void rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                            const float* __restrict__ w, TO* __restrict__ out, int d,
                                                            float eps) {
  constexpr int HOLD = 8;
  __shared__ float red[NW];
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * d;
  TO* o = out + (size_t)r * d;
  float ss = 0.f;
  const bool vec = (d & 3) == 0;
  const bool held = vec && d <= HOLD * 4 * NW * WAVE;
  float4 keep[HOLD];
  if (vec) {
    const float4* x4 = (const float4*)xr;
#pragma unroll
    for (int c = 0; c < HOLD; ++c) {
      const int i = threadIdx.x + c * NW * WAVE;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < d / 4) v = x4[i];
      keep[c] = v;
      ss += v.x * v.x;
      ss += v.y * v.y;
      ss += v.z * v.z;
      ss += v.w * v.w;
    }
    for (int i = threadIdx.x + HOLD * NW * WAVE; i < d / 4; i += NW * WAVE) {
      const float4 v = x4[i];
      ss += v.x * v.x;
      ss += v.y * v.y;
      ss += v.z * v.z;
      ss += v.w * v.w;
    }
  } else {
    for (int i = threadIdx.x; i < d; i += NW * WAVE) ss += xr[i] * xr[i];
  }
  ss = block_sum<NW>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)d + eps);
  if (held) {
#pragma unroll
    for (int c = 0; c < HOLD; ++c) {
      const int i = threadIdx.x + c * NW * WAVE;
      if (i < d / 4) {
        const float4 wv = ((const float4*)w)[i];
        const float a = keep[c].x * scale * wv.x, b = keep[c].y * scale * wv.y;
        const float e = keep[c].z * scale * wv.z, f = keep[c].w * scale * wv.w;
        if (sizeof(TO) == 4) {
          *(float4*)(o + 4 * i) = make_float4(a, b, e, f);
        } else {
          uint2 p;
          p.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
          p.y = (uint32_t)f32_to_bf16(e) | ((uint32_t)f32_to_bf16(f) << 16);
          *(uint2*)(o + 4 * i) = p;
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < d; i += NW * WAVE) Elem<TO>::store(o + i, xr[i] * scale * w[i]);
  }
}

extern "C" const char* dlgo_rmsnorm(const float* x, const int32_t* rows, const float* w, void* out, int out_dtype,
                                    int n_rows, int d, float eps, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && d > 0, "rmsnorm: bad sizes rows=%d d=%d", n_rows, d);
  DLGO_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
  DLGO_REQUIRE(d % 4 || ((((uintptr_t)x | (uintptr_t)w) & 15) == 0 && ((uintptr_t)out & (out_dtype == DLGO_DTYPE_F32 ? 15 : 7)) == 0),
               "rmsnorm: rows of a width that is a multiple of 4 must be 16-byte aligned");
  if (n_rows == 0) return nullptr;
  // the number of waves per row is a function of d alone
  const bool small = d <= 1024;
  if (out_dtype == DLGO_DTYPE_F32) {
    if (small) hipLaunchKernelGGL((rmsnorm_kernel<float, 1>), dim3(n_rows), dim3(WAVE), 0, stream, x, rows, w, (float*)out, d, eps);
    else hipLaunchKernelGGL((rmsnorm_kernel<float, 4>), dim3(n_rows), dim3(4 * WAVE), 0, stream, x, rows, w, (float*)out, d, eps);
  } else if (out_dtype == DLGO_DTYPE_BF16) {
    if (small) hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, 1>), dim3(n_rows), dim3(WAVE), 0, stream, x, rows, w, (bf16_t*)out, d, eps);
    else hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, 4>), dim3(n_rows), dim3(4 * WAVE), 0, stream, x, rows, w, (bf16_t*)out, d, eps);
  } else {
    DLGO_FAIL("rmsnorm: unknown dtype code %d", out_dtype);
  }
  DLGO_LAUNCH_CHECK("rmsnorm");
  return nullptr;
}

#include "exact_end.h"

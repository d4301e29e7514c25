// Two small steps that some attention layers put between the projections and the rotation, each a kernel of its own
// so that layers without them pay nothing (computerex/dlgo, models/llm/forward.go:227-244):
//   bias:         y[t, n] += b[n]                                   (ops.AddBias, :227-235)
//   per-head norm: every head of q and of k is RMS-normalised over its own elements with one weight vector
//                  of the head's size, x * (1/sqrt(mean(x^2) + eps)) * w                (:236-244)
// Sums and scales are float32 whatever the rows are stored in.
#include "common.h"
// everything here is float32 arithmetic whatever the storage type: no approximation can be named (exact_begin.h)
#include "exact_begin.h"

template <typename TY>
__global__ __launch_bounds__(256) void bias_add_kernel(TY* __restrict__ y, int ld, const float* __restrict__ b, int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  TY* p = y + (size_t)blockIdx.y * ld + n;
  Elem<TY>::store(p, Elem<TY>::load(p) + b[n]);
}

// one wave per (row, head); heads are hd consecutive elements starting at column col0 + head * hd
template <typename T>
__global__ __launch_bounds__(WAVE) void head_rmsnorm_kernel(T* __restrict__ x, int ld, int col0, int hd,
                                                            const float* __restrict__ w, float eps) {
  T* p = x + (size_t)blockIdx.y * ld + col0 + (size_t)blockIdx.x * hd;
  const int lane = threadIdx.x;
  float ss = 0.f;
  for (int i = lane; i < hd; i += WAVE) {
    const float v = Elem<T>::load(p + i);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float scale = 1.0f / sqrtf(ss / (float)hd + eps);
  for (int i = lane; i < hd; i += WAVE) Elem<T>::store(p + i, Elem<T>::load(p + i) * scale * w[i]);
}

// y [n_rows, N] (row stride ld, dtype code of its elements) += b [N] float32
extern "C" const char* dlgo_bias_add(void* y, int dtype, int n_rows, int N, int ld, const float* b, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && n_rows <= 65535 && N > 0 && ld >= N, "bias_add: bad sizes rows=%d N=%d ld=%d (at most 65535 rows)", n_rows, N, ld);
  DLGO_REQUIRE(y && b, "bias_add: missing argument");
  if (n_rows == 0) return nullptr;
  const dim3 grid((N + 255) / 256, n_rows);
  if (dtype == DLGO_DTYPE_F32) hipLaunchKernelGGL(bias_add_kernel<float>, grid, dim3(256), 0, stream, (float*)y, ld, b, N);
  else if (dtype == DLGO_DTYPE_BF16) hipLaunchKernelGGL(bias_add_kernel<bf16_t>, grid, dim3(256), 0, stream, (bf16_t*)y, ld, b, N);
  else DLGO_FAIL("bias_add: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("bias_add");
  return nullptr;
}

// heads col0/hd .. of each row of x [n_rows, ld] are normalised in place with weight w [hd] float32
extern "C" const char* dlgo_head_rmsnorm(void* x, int dtype, int n_rows, int ld, int col0, int n_heads, int hd, const float* w,
                                         float eps, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && n_rows <= 65535 && n_heads > 0 && hd > 0 && col0 >= 0 && col0 + n_heads * hd <= ld,
               "head_rmsnorm: bad sizes rows=%d heads=%d hd=%d col0=%d ld=%d (at most 65535 rows)", n_rows, n_heads, hd, col0, ld);
  DLGO_REQUIRE(x && w && eps > 0.f, "head_rmsnorm: missing argument or eps not positive");
  if (n_rows == 0) return nullptr;
  const dim3 grid(n_heads, n_rows);
  if (dtype == DLGO_DTYPE_F32) hipLaunchKernelGGL(head_rmsnorm_kernel<float>, grid, dim3(WAVE), 0, stream, (float*)x, ld, col0, hd, w, eps);
  else if (dtype == DLGO_DTYPE_BF16) hipLaunchKernelGGL(head_rmsnorm_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, (bf16_t*)x, ld, col0, hd, w, eps);
  else DLGO_FAIL("head_rmsnorm: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("head_rmsnorm");
  return nullptr;
}

#include "exact_end.h"

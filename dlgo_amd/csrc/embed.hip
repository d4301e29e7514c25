// Embedding gather: ids[T] -> x[T, d] in float32 (the residual stream is float32
// in both run dtypes).  computerex/dlgo copies one table row per token on the CPU
// even in GPU mode (core/tensor.go:40-57, gpu/forward.go:23-34) and drops the
// error of an id out of range (models/llm/forward.go:132-135); here the host
// rejects such ids before the launch and the kernel clamps so that it cannot fault.
#include "common.h"
// everything here is float32 arithmetic whatever the storage type: no approximation can be named (exact_begin.h)
#include "exact_begin.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                                    float* __restrict__ x, int d, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * d;
  float* out = x + (size_t)t * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = Elem<T>::load(row + i);
}

extern "C" const char* dlgo_embed(const void* table, int dtype, const int32_t* ids, float* x, int n_tokens, int d,
                                  int vocab, hipStream_t stream) {
  DLGO_REQUIRE(n_tokens >= 0 && d > 0 && vocab > 0, "embed: bad sizes T=%d d=%d vocab=%d", n_tokens, d, vocab);
  if (n_tokens == 0) return nullptr;
  if (dtype == DLGO_DTYPE_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, (const float*)table, ids, x, d, vocab);
  else if (dtype == DLGO_DTYPE_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, stream, (const bf16_t*)table, ids, x, d, vocab);
  else
    DLGO_FAIL("embed: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("embed");
  return nullptr;
}

#include "exact_end.h"

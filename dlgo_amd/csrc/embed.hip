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

// Rows by index, whatever they hold: dst[dst_rows[i]] = src[src_rows[i]] for i < n, a row being row_words 4-byte words
// (either list may be missing: then i itself).  What the loop and the cache need when the set of live sequences or a
// page table changes: rows of logits or ids picked out, page-table rows put in place, pages copied.  Source and
// destination rows must not overlap each other.
__global__ __launch_bounds__(256) void copy_rows_kernel(const uint32_t* __restrict__ src, const int32_t* __restrict__ src_rows,
                                                        uint32_t* __restrict__ dst, const int32_t* __restrict__ dst_rows,
                                                        long long row_words, long long ld_src, long long ld_dst, int vec) {
  const int i = blockIdx.y;
  const uint32_t* from = src + (size_t)(src_rows ? src_rows[i] : i) * ld_src;
  uint32_t* to = dst + (size_t)(dst_rows ? dst_rows[i] : i) * ld_dst;
  if (vec) {                             // rows and strides of whole 16 bytes, 16-byte aligned
    const long long n4 = row_words >> 2;
    for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < n4; w += (long long)gridDim.x * blockDim.x)
      ((uint4*)to)[w] = ((const uint4*)from)[w];
  } else {
    for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < row_words; w += (long long)gridDim.x * blockDim.x)
      to[w] = from[w];
  }
}

// n rows of row_bytes bytes (a multiple of 4); ld_*: bytes from a row to the next (multiples of 4); the lists hold row
// numbers that the caller has checked against the two tensors.
extern "C" const char* dlgo_copy_rows(const void* src, const int32_t* src_rows, void* dst, const int32_t* dst_rows, int n,
                                      long long row_bytes, long long ld_src_bytes, long long ld_dst_bytes, hipStream_t stream) {
  DLGO_REQUIRE(n >= 0 && n <= 65535 && row_bytes > 0, "copy_rows: bad sizes n=%d row_bytes=%lld (at most 65535 rows)", n, row_bytes);
  DLGO_REQUIRE(row_bytes % 4 == 0 && ld_src_bytes % 4 == 0 && ld_dst_bytes % 4 == 0 && ((uintptr_t)src & 3) == 0 && ((uintptr_t)dst & 3) == 0,
               "copy_rows: rows, strides and addresses must be multiples of 4 bytes");
  DLGO_REQUIRE(ld_src_bytes >= row_bytes && ld_dst_bytes >= row_bytes, "copy_rows: row strides shorter than a row");
  if (n == 0) return nullptr;
  const int vec = row_bytes % 16 == 0 && ld_src_bytes % 16 == 0 && ld_dst_bytes % 16 == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
  const long long units = vec ? row_bytes / 16 : row_bytes / 4;
  long long bx = (units + 256 * 4 - 1) / (256 * 4);            // about four units a thread
  if (bx < 1) bx = 1;
  if (bx > 1024) bx = 1024;
  hipLaunchKernelGGL(copy_rows_kernel, dim3((unsigned)bx, n), dim3(256), 0, stream, (const uint32_t*)src, src_rows, (uint32_t*)dst,
                     dst_rows, row_bytes / 4, ld_src_bytes / 4, ld_dst_bytes / 4, vec);
  DLGO_LAUNCH_CHECK("copy_rows");
  return nullptr;
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

// Rotary position encoding of the query and key heads of a step's tokens, fused
// with the write of the rotated keys and the values into the paged cache.
//
// Rotation of pair i at absolute position p, with cos/sin read from a table
// built in float64 on the host (models/llm/workers.go:147-171):
//   x0' = x0*cos - x1*sin ; x1' = x0*sin + x1*cos
// split-half pairs (v[i], v[i+rot/2]) or interleaved pairs (v[2i], v[2i+1])
// (ops/rope.go:21-31; gpu/shaders/rope.comp:21-66).  Keys are stored after the
// rotation, values as they are (models/llm/forward.go:246-257).
//
// Cache page (64 tokens) of one layer: keys [kv_head][token][hd], then values
// transposed [kv_head][hd][token], so that both attention products read
// 16-byte pieces along their reduction axis.
#include "common.h"

#define PAGE 64

template <typename T>
__global__ __launch_bounds__(WAVE) void rope_kv_kernel(T* __restrict__ qkv, int ld, int n_heads, int n_kv, int hd, int rot,
                                                       int interleaved, const float* __restrict__ cos_t,
                                                       const float* __restrict__ sin_t, const int32_t* __restrict__ positions,
                                                       const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
                                                       const int32_t* __restrict__ page_table, int max_pages,
                                                       T* __restrict__ cache, long long page_stride, long long v_off,
                                                       int write_kv) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;   // [0,H): query, [H,H+KV): key, [H+KV,H+2KV): value
  const int lane = threadIdx.x;
  const int pos = positions[t];
  T* src = qkv + (size_t)t * ld + (size_t)head * hd;
  const bool is_q = head < n_heads;
  const bool is_k = !is_q && head < n_heads + n_kv;

  T* kdst = nullptr;   // key row in the cache, or the value column base
  int in_page = 0;
  if (!is_q) {
    if (!write_kv) return;
    const int slot = slots[tok_seq[t]];
    const int page = page_table[(size_t)slot * max_pages + pos / PAGE];
    if (page < 0) return;   // the host reserves pages before the launch; never write through a hole
    in_page = pos % PAGE;
    const int kvh = is_k ? head - n_heads : head - n_heads - n_kv;
    if (is_k) kdst = cache + (size_t)page * page_stride + ((size_t)kvh * PAGE + in_page) * hd;
    else kdst = cache + v_off + (size_t)page * page_stride + (size_t)kvh * hd * PAGE + in_page;
  }

  if (!is_q && !is_k) {   // value: transposed copy
    for (int i = lane; i < hd; i += WAVE) kdst[(size_t)i * PAGE] = src[i];
    return;
  }
  const int half = rot / 2;
  const float* c = cos_t ? cos_t + (size_t)pos * half : nullptr;
  const float* s = sin_t ? sin_t + (size_t)pos * half : nullptr;
  T* dst = is_q ? src : kdst;
  for (int i = lane; i < half; i += WAVE) {
    const int i0 = interleaved ? 2 * i : i;
    const int i1 = interleaved ? 2 * i + 1 : i + half;
    float x0 = Elem<T>::load(src + i0), x1 = Elem<T>::load(src + i1);
    if (c) {
      const float cs = c[i], sn = s[i];
      const float y0 = x0 * cs - x1 * sn;
      const float y1 = x0 * sn + x1 * cs;
      x0 = y0;
      x1 = y1;
    }
    Elem<T>::store(dst + i0, x0);
    Elem<T>::store(dst + i1, x1);
  }
  if (is_k)   // the part of the head beyond the rotated width is copied
    for (int i = rot + lane; i < hd; i += WAVE) kdst[i] = src[i];
}

extern "C" const char* dlgo_rope_kv(void* qkv, int dtype, int n_tokens, int ld, int n_heads, int n_kv, int hd, int rot,
                                    int interleaved, const float* cos_t, const float* sin_t, int table_rows,
                                    const int32_t* positions, const int32_t* tok_seq, const int32_t* slots,
                                    const int32_t* page_table, int max_pages, void* cache, long long page_stride,
                                    long long v_off, int write_kv, hipStream_t stream) {
  DLGO_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv >= 0 && hd > 0, "rope_kv: bad sizes");
  DLGO_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv: rotated width %d must be even and at most head_dim %d", rot, hd);
  DLGO_REQUIRE(ld >= (n_heads + 2 * n_kv) * hd, "rope_kv: row stride %d shorter than the heads it holds", ld);
  DLGO_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_kv: cos and sin tables come together");
  DLGO_REQUIRE(cos_t == nullptr || table_rows > 0, "rope_kv: empty rotation table");
  DLGO_REQUIRE(!write_kv || (cache && page_table && slots && tok_seq && max_pages > 0), "rope_kv: cache arguments missing");
  if (n_tokens == 0) return nullptr;
  dim3 grid(n_tokens, n_heads + 2 * n_kv);
  if (dtype == DLGO_DTYPE_F32)
    hipLaunchKernelGGL(rope_kv_kernel<float>, grid, dim3(WAVE), 0, stream, (float*)qkv, ld, n_heads, n_kv, hd, rot, interleaved,
                       cos_t, sin_t, positions, tok_seq, slots, page_table, max_pages, (float*)cache, page_stride, v_off, write_kv);
  else if (dtype == DLGO_DTYPE_BF16)
    hipLaunchKernelGGL(rope_kv_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, (bf16_t*)qkv, ld, n_heads, n_kv, hd, rot, interleaved,
                       cos_t, sin_t, positions, tok_seq, slots, page_table, max_pages, (bf16_t*)cache, page_stride, v_off, write_kv);
  else
    DLGO_FAIL("rope_kv: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("rope_kv");
  return nullptr;
}

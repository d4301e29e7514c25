// Causal grouped-query attention of a step's query rows over the paged cache.
//
// For query head h of a token at absolute position p (computerex/dlgo,
// models/llm/forward.go:258-278; gpu/shaders/attention.comp:28-95):
//   kvh = h / (H / KV);  s_t = (q_h . K[t][kvh]) / sqrt(hd)  for t in [lo, p]
//   P = softmax(s);  o_h = sum_t P_t V[t][kvh]
// The causal mask is the loop bound, as in the reference: there is no mask
// tensor.  lo = 0, or p - window + 1 for a windowed mixer (layers/gqa.go:98-132).
// The keys of the step's own tokens are already in the cache when this runs
// (models/llm/forward_batch.go:143-207), so prompts, single tokens and
// continuations are the same computation.
//
// Cache rows outside [lo, p] are never used in arithmetic: a stale or
// non-finite value there cannot reach the result.
//
// HEAD_DIM is fixed at compile time (one library per head size).
//
// Kernels:
//   attn_rows_kernel   any dtype; one wave per (token, query head), online
//                      softmax page by page in float32.  The float32 path.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
#define PAGE 64

static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 512, "head sizes come in steps of 16, up to 512");

template <typename T> struct Vec16;   // a 16-byte piece of a row, as floats
template <> struct Vec16<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void load(const float* p, float* f) {
    const float4 v = *(const float4*)p;
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* f) {
    const uint4 u = *(const uint4*)p;
    f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
    f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
    f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
    f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
  }
};

template <typename T>
__global__ __launch_bounds__(WAVE) void attn_rows_kernel(const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo,
                                                         const int32_t* __restrict__ positions,
                                                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ page_table, int max_pages,
                                                         const T* __restrict__ cache, long long page_stride, long long v_off,
                                                         int group, int window, float scale) {
  constexpr int HD = HEAD_DIM;
  constexpr int E = Vec16<T>::E;
  constexpr int ND = (HD + WAVE - 1) / WAVE;
  __shared__ float qs[HD];
  __shared__ float ps[PAGE];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  const int slot = slots[tok_seq[t]];
  const int kvh = h / group;
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;

  const T* qrow = q + (size_t)t * ldq + (size_t)h * HD;
  for (int i = lane; i < HD; i += WAVE) qs[i] = Elem<T>::load(qrow + i) * scale;
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.f;

  for (int pg = lo / PAGE; pg <= pos / PAGE; ++pg) {
    const int page = page_table[(size_t)slot * max_pages + pg];
    if (page < 0) continue;   // cannot happen for positions the host has reserved
    const T* kpage = cache + (size_t)page * page_stride + (size_t)kvh * PAGE * HD;
    const T* vpage = cache + v_off + (size_t)page * page_stride + (size_t)kvh * HD * PAGE;
    const int key = pg * PAGE + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const T* krow = kpage + (size_t)lane * HD;
      float d = 0.f;
#pragma unroll
      for (int c = 0; c < HD; c += E) {
        float kf[E];
        Vec16<T>::load(krow + c, kf);
#pragma unroll
        for (int e = 0; e < E; ++e) d = fmaf(qs[c + e], kf[e], d);
      }
      s = d;
    }
    const float m_new = fmaxf(m, wave_max(s));   // every page in the range holds at least one valid key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // 0 on the first page (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    const int k_lo = lo - pg * PAGE > 0 ? lo - pg * PAGE : 0;
    const int k_hi = pos - pg * PAGE < PAGE - 1 ? pos - pg * PAGE : PAGE - 1;
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = lane + i * WAVE;
      if (d < HD) {
        const T* vrow = vpage + (size_t)d * PAGE;
        float a = acc[i] * alpha;
        for (int k = k_lo; k <= k_hi; ++k) a = fmaf(ps[k], Elem<T>::load(vrow + k), a);
        acc[i] = a;
      }
    }
  }
  T* orow = out + (size_t)t * ldo + (size_t)h * HD;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = lane + i * WAVE;
    if (d < HD) Elem<T>::store(orow + d, acc[i] * inv);
  }
}

extern "C" int dlgo_attention_head_dim() { return HEAD_DIM; }

// q: rows of the step [T, >= H*hd] (rotated); out [T, >= H*hd]; positions, tok_seq per token; slots per sequence.
extern "C" const char* dlgo_attention_rows(const void* q, int ldq, void* out, int ldo, int dtype, int n_tokens, int n_heads,
                                           int n_kv, int head_dim, const int32_t* positions, const int32_t* tok_seq,
                                           const int32_t* slots, const int32_t* page_table, int max_pages, const void* cache,
                                           long long page_stride, long long v_off, int window, float scale,
                                           hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
  DLGO_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad head counts H=%d KV=%d", n_heads, n_kv);
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim, "attention: row strides too short");
  DLGO_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window or page table width");
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(((uintptr_t)cache & 15) == 0 && page_stride % epc == 0 && v_off % epc == 0, "attention: cache pages must be 16-byte aligned");
  if (n_tokens == 0) return nullptr;
  dim3 grid(n_tokens, n_heads);
  const int group = n_heads / n_kv;
  if (dtype == DLGO_DTYPE_F32)
    hipLaunchKernelGGL(attn_rows_kernel<float>, grid, dim3(WAVE), 0, stream, (const float*)q, ldq, (float*)out, ldo, positions,
                       tok_seq, slots, page_table, max_pages, (const float*)cache, page_stride, v_off, group, window, scale);
  else if (dtype == DLGO_DTYPE_BF16)
    hipLaunchKernelGGL(attn_rows_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, positions,
                       tok_seq, slots, page_table, max_pages, (const bf16_t*)cache, page_stride, v_off, group, window, scale);
  else
    DLGO_FAIL("attention: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("attention_rows");
  return nullptr;
}

// Choosing the next token from float32 logits on the device, one block per row,
// so that no logits travel to the host (computerex/dlgo downloads all of them for
// every token and samples on the CPU, gpu/forward.go:126, gpu/pipeline.go:225,250).
//
// argmax: first maximum wins (ops/ops.go:272-285).
// sample: the reference's pipeline (ops/sampling.go:32-48), per row with its own
// options: repetition penalty (:53-69) -> temperature (:72-80) -> top-k (:83-95)
// -> top-p (:99-138) -> min-p (:143-165) -> softmax and inverse-CDF draw with a
// uniform number (:167-181).  exp is exact (the reference's softmax uses a
// polynomial, ops/ops.go:125-147).  Every reduction runs in a fixed order, so a
// row's token depends on its logits, options and uniform number only.
// Differences from the reference, both at ties only: values equal to the top-p
// cut are all kept (the reference's unstable sort keeps some of them), and a
// masked token is never drawn, not even for a uniform number of exactly 0.
#include "common.h"

#define SAMP_THREADS 1024
#define SAMP_WAVES (SAMP_THREADS / WAVE)

__device__ __forceinline__ uint32_t order_key(float f) {   // larger float <-> larger key
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct BestIdx {
  float v;
  int i;
};
__device__ __forceinline__ BestIdx better(BestIdx a, BestIdx b) {
  // larger value, then smaller index; NaN never wins
  if (b.i >= 0 && (a.i < 0 || b.v > a.v || (b.v == a.v && b.i < a.i))) return b;
  return a;
}

__device__ BestIdx block_argmax(const float* row, int V, BestIdx* red) {
  BestIdx best = {-INFINITY, -1};
  for (int i = threadIdx.x; i < V; i += SAMP_THREADS) {
    const float v = row[i];
    if (v == v) best = better(best, BestIdx{v, i});
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    BestIdx other;
    other.v = __shfl_xor(best.v, o, WAVE);
    other.i = __shfl_xor(best.i, o, WAVE);
    best = better(best, other);
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  BestIdx r = red[0];
  for (int w = 1; w < SAMP_WAVES; ++w) r = better(r, red[w]);
  return r;
}

__device__ float block_sum_f(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < SAMP_WAVES; ++w) t += red[w];
  return t;
}

// argmax in two stages, so that a few rows still fill the chip: ARGMAX_CHUNKS blocks per row each find the
// best of their part of the row, then one wave per row picks among them (larger value, then smaller index).
#define ARGMAX_CHUNKS 64
#define ARGMAX_THREADS 256

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_part_kernel(const float* __restrict__ logits, int ld, int V,
                                                                     BestIdx* __restrict__ partial) {
  __shared__ BestIdx red[ARGMAX_THREADS / WAVE];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
  const int b0 = chunk * per, b1 = b0 + per < V ? b0 + per : V;
  const float* lg = logits + (size_t)row * ld;
  BestIdx best = {-INFINITY, -1};
  for (int i = b0 + threadIdx.x; i < b1; i += ARGMAX_THREADS) {
    const float v = lg[i];
    if (v == v) best = better(best, BestIdx{v, i});
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    BestIdx other;
    other.v = __shfl_xor(best.v, o, WAVE);
    other.i = __shfl_xor(best.i, o, WAVE);
    best = better(best, other);
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    BestIdx r = red[0];
    for (int w = 1; w < ARGMAX_THREADS / WAVE; ++w) r = better(r, red[w]);
    partial[(size_t)row * ARGMAX_CHUNKS + chunk] = r;
  }
}

__global__ __launch_bounds__(WAVE) void argmax_final_kernel(const BestIdx* __restrict__ partial, int32_t* __restrict__ out) {
  BestIdx best = partial[(size_t)blockIdx.x * ARGMAX_CHUNKS + threadIdx.x];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    BestIdx other;
    other.v = __shfl_xor(best.v, o, WAVE);
    other.i = __shfl_xor(best.i, o, WAVE);
    best = better(best, other);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best.i < 0 ? 0 : best.i;
}

// Largest key tau with measure({i : key_i >= tau}) >= need, by bisection on the key's bits.
// COUNT: the measure counts elements (top-k); else it sums e_i (top-p).
template <bool COUNT>
__device__ uint32_t bisect_threshold(const float* work, const float* e, int V, float need, float* red) {
  uint32_t prefix = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t cand = prefix | (1u << bit);
    float part = 0.f;
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS)
      if (order_key(work[i]) >= cand) part += COUNT ? 1.0f : e[i];
    const float total = block_sum_f(part, red);
    if (total >= need) prefix = cand;
  }
  return prefix;
}

__global__ __launch_bounds__(SAMP_THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int V,
                                                              float* __restrict__ work_all, float* __restrict__ e_all,
                                                              const float* __restrict__ temperature,
                                                              const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                              const float* __restrict__ min_p, const float* __restrict__ penalty,
                                                              const int32_t* __restrict__ recent, int n_recent,
                                                              const float* __restrict__ uniform, int32_t* __restrict__ out) {
  __shared__ BestIdx redb[SAMP_WAVES];
  __shared__ float red[SAMP_WAVES];
  __shared__ float scan[SAMP_THREADS];
  __shared__ int chosen;
  const int row = blockIdx.x;
  const float* lg = logits + (size_t)row * ld;
  const float temp = temperature[row];
  if (!(temp > 0.f)) {   // greedy row
    const BestIdx b = block_argmax(lg, V, redb);
    if (threadIdx.x == 0) out[row] = b.i < 0 ? 0 : b.i;
    return;
  }
  float* work = work_all + (size_t)row * V;
  float* e = e_all + (size_t)row * V;
  const float inv_temp = temp == 1.0f ? 1.0f : 1.0f / temp;
  for (int i = threadIdx.x; i < V; i += SAMP_THREADS) work[i] = lg[i];
  __syncthreads();
  // repetition penalty: each distinct recent token once
  const float pen = penalty[row];
  if (pen > 1.0f && n_recent > 0 && (int)threadIdx.x < n_recent) {
    const int32_t* rc = recent + (size_t)row * n_recent;
    const int tok = rc[threadIdx.x];
    bool first = tok >= 0 && tok < V;
    for (int j = 0; first && j < (int)threadIdx.x; ++j) first = rc[j] != tok;
    if (first) work[tok] = work[tok] > 0.f ? work[tok] / pen : work[tok] * pen;
  }
  __syncthreads();
  if (inv_temp != 1.0f)
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS) work[i] *= inv_temp;
  __syncthreads();
  // top-k: everything below the k-th largest value is masked; ties at it stay
  const int k = top_k[row];
  if (k > 0 && k < V) {
    const uint32_t tau = bisect_threshold<true>(work, nullptr, V, (float)k, red);
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS)
      if (order_key(work[i]) < tau) work[i] = -INFINITY;
    __syncthreads();
  }
  BestIdx top = block_argmax(work, V, redb);
  // top-p: smallest set, by falling probability, whose mass reaches p
  const float tp = top_p[row];
  if (tp < 1.0f) {
    float part = 0.f;
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS) {
      const float v = expf(work[i] - top.v);
      e[i] = v;
      part += v;
    }
    __syncthreads();
    const float Z = block_sum_f(part, red);
    const uint32_t tau = bisect_threshold<false>(work, e, V, tp * Z, red);
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS)
      if (order_key(work[i]) < tau) work[i] = -INFINITY;
    __syncthreads();
  }
  // min-p: probability below min_p * (largest probability) is masked
  const float mp = min_p[row];
  if (mp > 0.f) {
    const float cut = top.v + logf(mp);
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS)
      if (work[i] < cut) work[i] = -INFINITY;
    __syncthreads();
  }
  // softmax and inverse-CDF draw, cumulative sums in index order
  const int chunk = (V + SAMP_THREADS - 1) / SAMP_THREADS;
  const int b0 = threadIdx.x * chunk, b1 = b0 + chunk < V ? b0 + chunk : V;
  float mine = 0.f;
  for (int i = b0; i < b1; ++i) {
    const float v = expf(work[i] - top.v);
    e[i] = v;
    mine += v;
  }
  scan[threadIdx.x] = mine;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  for (int o = 1; o < SAMP_THREADS; o <<= 1) {   // inclusive scan
    const float add = (int)threadIdx.x >= o ? scan[threadIdx.x - o] : 0.f;
    __syncthreads();
    scan[threadIdx.x] += add;
    __syncthreads();
  }
  const float Z = scan[SAMP_THREADS - 1];
  const float target = uniform[row] * Z;
  const float incl = scan[threadIdx.x], excl = threadIdx.x ? scan[threadIdx.x - 1] : 0.f;
  if (mine > 0.f && (excl < target || (threadIdx.x == 0 && target <= 0.f)) && target <= incl) {
    float cum = excl;
    int pick = -1, last = -1;
    for (int i = b0; i < b1; ++i) {
      if (e[i] > 0.f) {
        cum += e[i];
        last = i;
        if (cum >= target) {
          pick = i;
          break;
        }
      }
    }
    chosen = pick >= 0 ? pick : last;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[row] = chosen >= 0 ? chosen : (top.i < 0 ? 0 : top.i);
}

// partial: scratch of n_rows * 64 pairs (float, int32), 8 bytes each.
extern "C" const char* dlgo_argmax(const float* logits, int ld, int n_rows, int V, void* partial, long long partial_bytes,
                                   int32_t* out, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
  DLGO_REQUIRE(n_rows <= 65535, "argmax: at most 65535 rows at a time");
  DLGO_REQUIRE(partial && partial_bytes >= (long long)n_rows * ARGMAX_CHUNKS * (long long)sizeof(BestIdx), "argmax: scratch too small");
  static_assert(ARGMAX_CHUNKS == WAVE, "the final stage reads one candidate per lane");
  if (n_rows == 0) return nullptr;
  hipLaunchKernelGGL(argmax_part_kernel, dim3(ARGMAX_CHUNKS, n_rows), dim3(ARGMAX_THREADS), 0, stream, logits, ld, V, (BestIdx*)partial);
  DLGO_LAUNCH_CHECK("argmax");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(WAVE), 0, stream, (const BestIdx*)partial, out);
  DLGO_LAUNCH_CHECK("argmax");
  return nullptr;
}

// work and e: [n_rows, V] float32 scratch.  recent: [n_rows, n_recent] token ids, -1 where empty.
extern "C" const char* dlgo_sample(const float* logits, int ld, int n_rows, int V, float* work, float* e,
                                   const float* temperature, const int32_t* top_k, const float* top_p, const float* min_p,
                                   const float* penalty, const int32_t* recent, int n_recent, const float* uniform,
                                   int32_t* out, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
  DLGO_REQUIRE(n_recent >= 0 && n_recent <= SAMP_THREADS, "sample: at most %d recent tokens, got %d", SAMP_THREADS, n_recent);
  DLGO_REQUIRE(work && e && temperature && top_k && top_p && min_p && penalty && uniform && out, "sample: missing argument");
  DLGO_REQUIRE(n_recent == 0 || recent, "sample: recent tokens missing");
  if (n_rows == 0) return nullptr;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMP_THREADS), 0, stream, logits, ld, V, work, e, temperature, top_k, top_p,
                     min_p, penalty, recent, n_recent, uniform, out);
  DLGO_LAUNCH_CHECK("sample");
  return nullptr;
}

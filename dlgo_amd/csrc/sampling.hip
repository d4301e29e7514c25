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
#include "sampling.h"
#include <stddef.h>
#include <mutex>
// everything here is float32 arithmetic whatever the storage type: no approximation can be named (exact_begin.h)
#include "exact_begin.h"

#define SAMP_THREADS 1024
#define SAMP_WAVES (SAMP_THREADS / WAVE)

__device__ __forceinline__ uint32_t order_key(float f) {   // larger float <-> larger key; -0 and +0 are one value
  const uint32_t u = __float_as_uint(f + 0.0f);              // -0 + 0 = +0
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

// f(index, value) for every element of a row, the block's threads striding over it; 16 bytes a thread at a time, and
// several of them on their way at once, where the row allows (vec).
template <typename F>
__device__ __forceinline__ void for_each_element(const float* __restrict__ row, int V, bool vec, F f) {
  if (vec) {
    const float4* r4 = (const float4*)row;
#pragma unroll 8
    for (int i = threadIdx.x; i < V / 4; i += SAMP_THREADS) {
      const float4 x = r4[i];
      f(4 * i, x.x);
      f(4 * i + 1, x.y);
      f(4 * i + 2, x.z);
      f(4 * i + 3, x.w);
    }
  } else {
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS) f(i, row[i]);
  }
}

// the best of what the block's threads have each found
__device__ BestIdx block_best(BestIdx best, BestIdx* red) {
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

__device__ BestIdx block_argmax(const float* row, int V, BestIdx* red, bool vec = false) {
  BestIdx best = {-INFINITY, -1};
  for_each_element(row, V, vec, [&](int i, float v) {
    if (v == v) best = better(best, BestIdx{v, i});
  });
  return block_best(best, red);
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

// Largest key tau with |{i : key_i >= tau}| >= need (top-k), found 11, 11 and 10 bits of the key at a time, each time
// from a count of the elements by those bits: three passes over the row.  hist: 2048 ints of LDS; at: two ints of LDS.
// Called by the whole block.
__device__ uint32_t radix_threshold(const float* work, int V, int need, int* hist, int* at, bool vec) {
  uint32_t prefix = 0;              // the key's upper bits, as far as they are known
  for (int level = 0; level < 3; ++level) {
    const int shift = level == 0 ? 21 : (level == 1 ? 10 : 0), bits = level == 2 ? 10 : 11;
    for (int b = threadIdx.x; b < 2048; b += SAMP_THREADS) hist[b] = 0;
    __syncthreads();
    for_each_element(work, V, vec, [&](int, float x) {
      const uint32_t key = order_key(x);
      if (level == 0 || (key >> (shift + bits)) == prefix) atomicAdd(&hist[(key >> shift) & ((1u << bits) - 1u)], 1);
    });
    __syncthreads();
    if (threadIdx.x < WAVE) {
      // the highest bin from which upwards `need` elements lie: a lane adds up 32 neighbouring bins, the lanes are
      // added from the top, and the lane in whose bins the count is reached walks them down
      const int lane = threadIdx.x;
      int mine = 0;
      for (int q = 0; q < 32; ++q) mine += hist[32 * lane + q];
      int from_top = mine;          // this lane's bins and all above
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const int y = __shfl_down(from_top, o, WAVE);
        if (lane + o < WAVE) from_top += y;
      }
      const unsigned long long reached = __ballot(from_top >= need);
      // (not reached at all: fewer elements than asked for share the prefix, which cannot be: the level above counted
      // them; at the first level it means fewer than `need` elements in the row, and every element stays)
      const int owner = reached ? 63 - __clzll(reached) : 0;
      if (lane == owner) {
        int above = from_top - mine, bin = 32 * lane;
        for (int q = 31; q >= 0; --q) {
          if (above + hist[32 * lane + q] >= need || q == 0) {
            bin = 32 * lane + q;
            break;
          }
          above += hist[32 * lane + q];
        }
        at[0] = bin;
        at[1] = above;
      }
    }
    __syncthreads();
    prefix = (prefix << bits) | (uint32_t)at[0];
    need -= at[1];
    __syncthreads();
  }
  return prefix;
}

// The candidates of a row after top-k, when they are few enough to sit in LDS one to a thread: the exact top-k cut, top-p,
// min-p and the draw, all in index order.  cv/ci hold n candidates in any order; every element outside them is masked.
#define SAMP_CAND SAMP_THREADS
struct SampleSmall {
  float cv[SAMP_CAND];
  int ci[SAMP_CAND];
  float sv[SAMP_CAND];
  int si[SAMP_CAND];
  float se[SAMP_CAND];
  uint32_t skey[SAMP_CAND];
  float scan[SAMP_THREADS];
  int n, first, last;
  uint32_t tau;
};

__device__ int sample_small(SampleSmall& S, int n, int k, BestIdx top, float tp, float mp, float u) {
  const int j = threadIdx.x;
  const bool have = j < n;
  // into index order
  const int my_i0 = have ? S.ci[j] : 0x7fffffff;
  const float my_v0 = have ? S.cv[j] : -INFINITY;
  int pos = 0;
  for (int i = 0; i < n; ++i) pos += S.ci[i] < my_i0;
  if (have) {
    S.sv[pos] = my_v0;
    S.si[pos] = my_i0;
  }
  if (j == 0) {
    S.first = 0x7fffffff;
    S.last = -1;
    S.tau = 0;
  }
  __syncthreads();
  const float v = have ? S.sv[j] : -INFINITY;
  const uint32_t key = order_key(v);
  S.skey[j] = have ? key : 0u;
  __syncthreads();
  // top-k: an element stays if fewer than k are strictly larger (ties at the cut all stay)
  int rank = 0;
  for (int i = 0; i < n; ++i) rank += S.skey[i] > key;
  bool keep = have && rank < k;
  float e = keep ? expf(v - top.v) : 0.f;
  if (tp < 1.0f) {      // top-p: the largest cut whose elements at or above it hold p of the mass
    S.se[j] = e;
    __syncthreads();
    float Z = 0.f, mass = 0.f;
    for (int i = 0; i < n; ++i) {
      const float ei = S.se[i];
      Z += ei;
      if (S.skey[i] >= key) mass += ei;
    }
    if (keep && mass >= tp * Z) atomicMax(&S.tau, key);
    __syncthreads();
    keep = keep && key >= S.tau;
  }
  if (mp > 0.f) keep = keep && !(v < top.v + logf(mp));
  e = keep ? e : 0.f;
  // inverse-CDF draw over the cumulative sums in index order
  S.scan[j] = e;
  __syncthreads();
  for (int o = 1; o < SAMP_THREADS; o <<= 1) {
    const float add = j >= o ? S.scan[j - o] : 0.f;
    __syncthreads();
    S.scan[j] += add;
    __syncthreads();
  }
  const float target = u * S.scan[SAMP_THREADS - 1];
  if (e > 0.f) {
    if (S.scan[j] >= target) atomicMin(&S.first, j);
    atomicMax(&S.last, j);
  }
  __syncthreads();
  const int pick = S.first != 0x7fffffff ? S.first : S.last;
  return pick >= 0 ? S.si[pick] : (top.i < 0 ? 0 : top.i);
}

// The first of the 255 bins of `hist` at which the running count reaches k, found by the block's first wave (four bins
// a lane, a scan over the lanes, then the lane's own four): *bin = that bin or 255 if none does, *cum = the count up to
// and including it (all of them if none does).  Every thread of wave 0 must call it; the results are in lane 0.
__device__ __forceinline__ void first_bin_reaching(const int* hist, int k, int* bin, int* cum) {
  const int lane = threadIdx.x & 63;
  int h[4], mine = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    h[q] = 4 * lane + q < 255 ? hist[4 * lane + q] : 0;
    mine += h[q];
  }
  int incl = mine;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const int y = __shfl_up(incl, o, WAVE);
    if (lane >= o) incl += y;
  }
  const unsigned long long hit = __ballot(incl >= k);
  const int total = __shfl(incl, WAVE - 1, WAVE);
  if (!hit) {
    *bin = 255;
    *cum = total;
    return;
  }
  const int owner = __ffsll((long long)hit) - 1;
  int c = __shfl(incl - mine, owner, WAVE), b = 4 * owner;
  const int h0 = __shfl(h[0], owner, WAVE), h1 = __shfl(h[1], owner, WAVE), h2 = __shfl(h[2], owner, WAVE), h3 = __shfl(h[3], owner, WAVE);
  const int hs[4] = {h0, h1, h2, h3};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    c += hs[q];
    if (c >= k) {
      b += q;
      break;
    }
  }
  *bin = b;
  *cum = c;
}

// Rows with a small top-k (the reference's default options have 40) need not be walked by one block: whatever survives
// top-k is among the largest k of its part of the row.  topk_part_kernel: TK_CHUNKS blocks a row; each keeps its part
// of the row (with temperature and penalty applied) in LDS, finds the part's maximum and, by the same count of
// distances below it as sample_kernel uses, a set of at most TK_CAP elements that holds the part's k largest (with
// everything tied at the k-th), and leaves them in the row's scratch.  topk_final_kernel: one block a row gathers the
// parts' sets, cuts them down the same way against the row's maximum and hands them to sample_small, which makes the
// exact cuts and the draw.  An element that is missing from a part's set has k larger ones in its own part, so it is
// below the k-th value of the row: the set that sample_small ends up with is the one sample_kernel would have had.
// A row that nothing cuts (no top-k, top-p or min-p) goes the same way with sums in place of candidates (see
// whole_row_draw), and a row whose only cut is min-p with the elements near its parts' maxima as candidates (see
// min_p_row), as has a row with a top-k between TK_CAP and SAMP_CAND (see large_top_k).  Whatever does not fit (a part
// with more than TK_CAP elements within its cut, no cut within 255 steps, a row with top-p but no top-k, a larger
// top-k still) is left to sample_kernel: the row's scratch says which rows are done.
// The row's scratch (floats of its row of `work`): maxima [TK_CHUNKS] as (value, index), counts [TK_CHUNKS] (-1: this
// part gave up), the done flag, then the parts' values [TK_CHUNKS][TK_CAP] and indices [TK_CHUNKS][TK_CAP] (for a row
// that nothing cuts: counts = the part's pieces of 256, values = their masses).
#define TK_CHUNKS 32
#define TK_CAP 128
#define TK_THREADS 256
#define TK_CHUNK_MAX 8192                      // floats of a part that LDS takes: rows of up to 262,144
#define TK_MIN_V 16384
#define TK_COUNTS (2 * TK_CHUNKS)
#define TK_DONE (3 * TK_CHUNKS)
#define TK_VALUES 128
#define TK_INDICES (TK_VALUES + TK_CHUNKS * TK_CAP)
#define TK_SCRATCH (TK_INDICES + TK_CHUNKS * TK_CAP)

// the elements of a part of a row (the last part may be shorter)
__device__ __forceinline__ int part_length(int V) { return ((V + TK_CHUNKS - 1) / TK_CHUNKS + 3) & ~3; }

// A row that is drawn from as it is, but for temperature and penalty: no top-k, top-p or min-p cuts anything.  Such a
// row needs no candidates, only sums, and those the parts can make as well.
__device__ __forceinline__ bool whole_row_draw(float temp, int k, float tp, float mp, int V) {
  return temp > 0.f && (k <= 0 || k >= V) && !(tp < 1.0f) && !(mp > 0.f);
}

// A row whose only cut is min-p: what stays lies within log(min_p) of the row's maximum, so within that of its
// part's maximum, and a part can offer those elements as it offers the largest k.
__device__ __forceinline__ bool min_p_row(float temp, int k, float tp, float mp, int V) {
  return temp > 0.f && (k <= 0 || k >= V) && !(tp < 1.0f) && mp > 0.f;
}

// A top-k of more than TK_CAP and at most SAMP_CAND: a part cannot offer its largest k, but it can offer its largest
// TK_CAP as for min_p_row, and topk_final_kernel can tell whether the row's largest k lie among what it was offered
// (each part's smallest offer falls below them).
__device__ __forceinline__ bool large_top_k(float temp, int k, int V) { return temp > 0.f && k > TK_CAP && k <= SAMP_CAND && k < V; }

__global__ __launch_bounds__(TK_THREADS) void topk_part_kernel(const float* __restrict__ logits, int ld, int V,
                                                               float* __restrict__ work_all,
                                                               const float* __restrict__ temperature,
                                                               const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                               const float* __restrict__ min_p, const float* __restrict__ penalty,
                                                               const int32_t* __restrict__ recent, int n_recent,
                                                               const int32_t* __restrict__ recent_rows,
                                                               const int32_t* __restrict__ counts) {
  __shared__ float xs[TK_CHUNK_MAX];
  __shared__ BestIdx red[TK_THREADS / WAVE];
  __shared__ int hist[256];
  __shared__ int limit, n_kept;
  __shared__ int rcs[SAMP_THREADS];               // the row's recent tokens
  const int row = blockIdx.y, chunk = blockIdx.x;
  float* scratch = work_all + (size_t)row * V;
  int* cnt = (int*)scratch + TK_COUNTS;
  if (chunk == 0 && threadIdx.x == 0) ((int*)scratch)[TK_DONE] = 0;
  const float temp = temperature[row];
  const int k = top_k[row];
  const bool whole = whole_row_draw(temp, k, top_p[row], min_p[row], V);
  // (the part's largest elements are what it offers of a row cut by min-p alone and of a row with a large top-k)
  const bool by_min_p = min_p_row(temp, k, top_p[row], min_p[row], V) || large_top_k(temp, k, V);
  if (!whole && !by_min_p && (!(temp > 0.f) || k < 1 || k > TK_CAP)) {       // not a row for this way
    if (threadIdx.x == 0) cnt[chunk] = -1;
    return;
  }
  const int per = part_length(V);
  const int c0 = chunk * per < V ? chunk * per : V, c1 = c0 + per < V ? c0 + per : V;
  const float* lg = logits + (size_t)row * ld;
  const float inv_temp = temp == 1.0f ? 1.0f : 1.0f / temp;
  // the part into LDS, every load on its way before the first is used where the row allows 16-byte loads
  if ((ld & 3) == 0 && ((uintptr_t)logits & 15) == 0 && ((c1 - c0) & 3) == 0) {
    const float4* src = (const float4*)(lg + c0);
    const int n4 = (c1 - c0) >> 2;
    constexpr int U = TK_CHUNK_MAX / 4 / TK_THREADS;       // 8
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = u * TK_THREADS + threadIdx.x;
      v[u] = i < n4 ? src[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = u * TK_THREADS + threadIdx.x;
      if (i < n4) {
        float4 x = v[u];
        if (inv_temp != 1.0f) {
          x.x *= inv_temp;
          x.y *= inv_temp;
          x.z *= inv_temp;
          x.w *= inv_temp;
        }
        ((float4*)xs)[i] = x;
      }
    }
  } else {
    for (int i = c0 + threadIdx.x; i < c1; i += TK_THREADS) xs[i - c0] = inv_temp != 1.0f ? lg[i] * inv_temp : lg[i];
  }
  if (threadIdx.x < 256) hist[threadIdx.x] = 0;
  // repetition penalty: each distinct recent token once, as in sample_kernel (the list is looked through in LDS)
  const float pen = penalty[row];
  const int rr = recent_rows ? recent_rows[row] : row;
  const int held = counts ? (counts[rr] < n_recent ? counts[rr] : n_recent) : n_recent;
  const bool penalised = pen > 1.0f && n_recent > 0;
  if (penalised)
    for (int t = threadIdx.x; t < held; t += TK_THREADS) rcs[t] = recent[(size_t)rr * n_recent + t];
  __syncthreads();
  if (penalised) {
    const int* rc = rcs;
    for (int t = threadIdx.x; t < held; t += TK_THREADS) {
      const int tok = rc[t];
      bool first = tok >= c0 && tok < c1;
      for (int j = 0; first && j < t; ++j) first = rc[j] != tok;
      if (first) {
        const float x = lg[tok] > 0.f ? lg[tok] / pen : lg[tok] * pen;
        xs[tok - c0] = inv_temp != 1.0f ? x * inv_temp : x;
      }
    }
  }
  __syncthreads();
  BestIdx best = {-INFINITY, -1};
  for (int i = c0 + threadIdx.x; i < c1; i += TK_THREADS) {
    const float v = xs[i - c0];
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
  best = red[0];
  for (int w = 1; w < TK_THREADS / WAVE; ++w) best = better(best, red[w]);
  if (best.i < 0) {                               // an empty part, or nothing but NaN: nothing to offer
    if (threadIdx.x == 0) {
      cnt[chunk] = 0;
      ((BestIdx*)scratch)[chunk] = best;
    }
    return;
  }
  if (whole) {
    // no cut at all: what the draw needs of this part is its mass, exp(x - the part's maximum) added up in pieces of
    // 256 elements (a lane four neighbours, then the lanes in a fixed order); topk_final_kernel scales the parts to the
    // row's maximum, finds the piece that reaches the target and walks that piece alone
    float* mass = scratch + TK_VALUES + chunk * TK_CAP;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_pieces = (c1 - c0 + 4 * WAVE - 1) / (4 * WAVE);
    for (int pc = wave; pc < n_pieces; pc += TK_THREADS / WAVE) {
      const int j0 = pc * 4 * WAVE + 4 * lane;
      float ev[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float below = j0 + e < c1 - c0 ? xs[j0 + e] - best.v : -INFINITY;
        ev[e] = below == below ? expf(below) : 0.f;        // (a part of nothing but -inf has no mass: -inf - -inf is no number)
      }
      float sum = ((ev[0] + ev[1]) + ev[2]) + ev[3];
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) sum += __shfl_xor(sum, o, WAVE);
      if (lane == 0) mass[pc] = sum;
    }
    if (threadIdx.x == 0) {
      cnt[chunk] = n_pieces;
      ((BestIdx*)scratch)[chunk] = best;
    }
    return;
  }
  if (by_min_p && best.v == -INFINITY) {          // a part of nothing but -inf offers nothing
    if (threadIdx.x == 0) {
      cnt[chunk] = 0;
      ((BestIdx*)scratch)[chunk] = best;
    }
    return;
  }
  const uint32_t kmax = order_key(best.v);
  for (int i = c0 + threadIdx.x; i < c1; i += TK_THREADS) {
    const uint32_t bin = (kmax - order_key(xs[i - c0])) >> 16;
    if (bin < 255u) atomicAdd(&hist[bin], 1);
  }
  __syncthreads();
  if (threadIdx.x < WAVE) {
    // the distance within which the k largest lie; if they do not lie within 255 steps, everything that does.
    // A row cut by min-p alone: the part cannot know the cut, which hangs on the row's maximum, so it offers its
    // largest elements, as many whole steps of distance as TK_CAP elements fill.  What it does not offer is smaller
    // than all it offers, so topk_final_kernel can tell whether anything that stays may be missing.
    int cum, b;
    first_bin_reaching(hist, by_min_p ? TK_CAP + 1 : k, &b, &cum);
    if (threadIdx.x == 0) {
      if (by_min_p) limit = b < 255 ? b - 1 : 254;
      else limit = cum <= TK_CAP ? (b < 255 ? b : 254) : -1;
      n_kept = 0;
    }
  }
  __syncthreads();
  if (limit < 0) {
    if (threadIdx.x == 0) cnt[chunk] = -1;
    return;
  }
  float* cv = scratch + TK_VALUES + chunk * TK_CAP;
  int* ci = (int*)scratch + TK_INDICES + chunk * TK_CAP;
  for (int i = c0 + threadIdx.x; i < c1; i += TK_THREADS) {
    const float x = xs[i - c0];
    if (((kmax - order_key(x)) >> 16) <= (uint32_t)limit) {
      const int slot = atomicAdd(&n_kept, 1);
      cv[slot] = x;
      ci[slot] = i;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    cnt[chunk] = n_kept;
    ((BestIdx*)scratch)[chunk] = best;
  }
}

__global__ __launch_bounds__(SAMP_THREADS) void topk_final_kernel(const float* __restrict__ logits, int ld, int V,
                                                                  float* __restrict__ work_all,
                                                                  const float* __restrict__ temperature,
                                                                  const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                                  const float* __restrict__ min_p, const float* __restrict__ penalty,
                                                                  int32_t* __restrict__ recent,
                                                                  int n_recent, const int32_t* __restrict__ recent_rows,
                                                                  int32_t* __restrict__ counts, const float* __restrict__ uniform,
                                                                  int32_t* __restrict__ out) {
  __shared__ SampleSmall S;
  __shared__ int hist[256];
  __shared__ int bstar, part_n[TK_CHUNKS];
  __shared__ BestIdx top_s;
  const int row = blockIdx.x;
  float* scratch = work_all + (size_t)row * V;
  const float temp = temperature[row];
  const int k = top_k[row];
  const bool whole = whole_row_draw(temp, k, top_p[row], min_p[row], V);
  const bool by_min_p = min_p_row(temp, k, top_p[row], min_p[row], V);
  const bool big_k = large_top_k(temp, k, V);
  if (!whole && !by_min_p && !big_k && (!(temp > 0.f) || k < 1 || k > TK_CAP)) return;
  __shared__ BestIdx part_top[TK_CHUNKS];
  __shared__ uint32_t least[TK_CHUNKS];             // the parts' smallest offers, as ordered keys
  if (threadIdx.x < TK_CHUNKS) least[threadIdx.x] = 0xffffffffu;
  if (threadIdx.x < TK_CHUNKS) {
    part_n[threadIdx.x] = ((const int*)scratch)[TK_COUNTS + threadIdx.x];
    part_top[threadIdx.x] = ((const BestIdx*)scratch)[threadIdx.x];
  }
  if (threadIdx.x < 256) hist[threadIdx.x] = 0;
  __syncthreads();
  if (threadIdx.x < WAVE) {
    const int c = threadIdx.x;
    BestIdx top = c < TK_CHUNKS && part_n[c] > 0 ? part_top[c] : BestIdx{-INFINITY, -1};
    const bool gave_up = c < TK_CHUNKS && part_n[c] < 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      BestIdx other;
      other.v = __shfl_xor(top.v, o, WAVE);
      other.i = __shfl_xor(top.i, o, WAVE);
      top = better(top, other);
    }
    const bool ok = __ballot(gave_up) == 0ull;
    if (threadIdx.x == 0) {
      top_s = top;
      bstar = ok && top.i >= 0 ? 0 : -2;
      S.n = 0;
    }
  }
  __syncthreads();
  if (bstar == -2) return;                        // a part gave up, or the row has nothing but NaN
  const BestIdx top = top_s;
  if (whole) {
    // The draw over the whole row from the parts' masses: one wave.  Cumulative sums in index order: the parts (each
    // scaled from its own maximum to the row's), within the part that reaches the target its pieces of 256, within
    // that piece its elements, taken from the logits again with temperature and penalty as the part applied them.
    // Where rounding leaves a level without an element that reaches the target, the last one with any weight is taken
    // (as sample_kernel does); a level with no weight at all leaves the row to sample_kernel.
    if (threadIdx.x >= WAVE) return;
    const int lane = threadIdx.x;
    auto scan64 = [&](float x) {          // inclusive, lanes in order
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float y = __shfl_up(x, o, WAVE);
        if (lane >= o) x += y;
      }
      return x;
    };
    auto first_reaching = [&](float weight, float incl, float before, float target, int* at, float* excl_at) {
      const unsigned long long hit = __ballot(weight > 0.f && before + incl >= target);
      const unsigned long long any = __ballot(weight > 0.f);
      if (!any) return false;
      *at = hit ? __ffsll((long long)hit) - 1 : 63 - __clzll(any);
      float excl = __shfl_up(incl, 1, WAVE);
      if (lane == 0) excl = 0.f;
      *excl_at = __shfl(excl, *at, WAVE);
      return true;
    };
    const int n_mine = lane < TK_CHUNKS ? part_n[lane] : 0;
    const float scale = n_mine > 0 ? expf(part_top[lane].v - top.v) : 0.f;
    float part_mass = 0.f;
    {
      const float* mass = scratch + TK_VALUES + (lane < TK_CHUNKS ? lane : 0) * TK_CAP;
      for (int pc = 0; pc < n_mine; ++pc) part_mass += mass[pc] * scale;
    }
    const float part_incl = scan64(part_mass);
    const float Z = __shfl(part_incl, WAVE - 1, WAVE);
    const float target = uniform[row] * Z;
    int c_at, p_at;
    float before, more;
    if (!first_reaching(part_mass, part_incl, 0.f, target, &c_at, &before)) return;
    const int n_pieces = __shfl(n_mine, c_at, WAVE);
    const float scale_at = __shfl(scale, c_at, WAVE);
    const float piece_mass = lane < n_pieces ? (scratch + TK_VALUES + c_at * TK_CAP)[lane] * scale_at : 0.f;
    if (!first_reaching(piece_mass, scan64(piece_mass), before, target, &p_at, &more)) return;
    before += more;
    // the piece's elements
    const int per = part_length(V);
    const int c0 = c_at * per, c1 = c0 + per < V ? c0 + per : V;
    const int i0 = c0 + p_at * 4 * WAVE + 4 * lane;
    const float* lg = logits + (size_t)row * ld;
    const float inv_temp = temp == 1.0f ? 1.0f : 1.0f / temp;
    const float pen = penalty[row];
    const int rr = recent_rows ? recent_rows[row] : row;
    const int held = counts ? (counts[rr] < n_recent ? counts[rr] : n_recent) : n_recent;
    const int32_t* rc = recent + (size_t)rr * n_recent;
    // which of the piece's elements are recent tokens: the list 64 at a time, a lane each, and passed round
    bool listed[4] = {false, false, false, false};
    if (pen > 1.0f && n_recent > 0) {
      const int piece0 = c0 + p_at * 4 * WAVE;
      for (int t0 = 0; t0 < held; t0 += WAVE) {
        const int mine_tok = t0 + lane < held ? rc[t0 + lane] : -1;
        const int m = held - t0 < WAVE ? held - t0 : WAVE;
        for (int t = 0; t < m; ++t) {
          const int tok = __shfl(mine_tok, t, WAVE);
          if ((unsigned)(tok - piece0) < (unsigned)(4 * WAVE)) {
#pragma unroll
            for (int e = 0; e < 4; ++e) listed[e] = listed[e] || tok == i0 + e;
          }
        }
      }
    }
    float ev[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ev[e] = 0.f;
      if (i0 + e < c1) {
        float x = lg[i0 + e];
        if (listed[e]) x = x > 0.f ? x / pen : x * pen;
        if (inv_temp != 1.0f) x *= inv_temp;
        ev[e] = expf(x - top.v);
      }
    }
    const float s1 = ev[0], s2 = s1 + ev[1], s3 = s2 + ev[2], s4 = s3 + ev[3];
    const float incl = scan64(s4);
    float excl = __shfl_up(incl, 1, WAVE);
    if (lane == 0) excl = 0.f;
    const float base = before + excl;
    const float sums[4] = {s1, s2, s3, s4};
    int mine_pick = -1, mine_last = -1;
#pragma unroll
    for (int e = 3; e >= 0; --e)
      if (ev[e] > 0.f) {
        if (mine_last < 0) mine_last = i0 + e;
        if (base + sums[e] >= target) mine_pick = i0 + e;
      }
    const unsigned long long hit = __ballot(mine_pick >= 0);
    const unsigned long long any = __ballot(mine_last >= 0);
    if (!any) return;
    const int pick = hit ? __shfl(mine_pick, __ffsll((long long)hit) - 1, WAVE) : __shfl(mine_last, 63 - __clzll(any), WAVE);
    if (lane == 0) {
      out[row] = pick;
      if (counts && n_recent > 0) {
        recent[(size_t)rr * n_recent + counts[rr] % n_recent] = pick;
        counts[rr] += 1;
      }
      ((int*)scratch)[TK_DONE] = 1;
    }
    return;
  }
  const uint32_t kmax = order_key(top.v);
  const float* cv = scratch + TK_VALUES;
  const int* ci = (const int*)scratch + TK_INDICES;
  // the thread's share of what the parts offer, asked for at once: slots threadIdx.x, + 1024, ...
  constexpr int PER = TK_CHUNKS * TK_CAP / SAMP_THREADS;
  float mine_v[PER];
  int mine_i[PER];
  bool mine[PER];
#pragma unroll
  for (int q = 0; q < PER; ++q) {
    const int e = q * SAMP_THREADS + threadIdx.x;
    mine[q] = (e % TK_CAP) < part_n[e / TK_CAP];
    mine_v[q] = mine[q] ? cv[e] : 0.f;
    mine_i[q] = mine[q] ? ci[e] : 0;
  }
  if (by_min_p) {
    // Of what the parts offer, what the cut against the row's maximum leaves (sample_small makes the same cut again),
    // if sample_small has room for it.  A part's offer is complete above its smallest element: if that one stays too,
    // smaller ones that the part kept to itself might, and the row is left to sample_kernel.
    const float cut = top.v + logf(min_p[row]);
#pragma unroll
    for (int q = 0; q < PER; ++q)
      if (mine[q]) atomicMin(&least[(q * SAMP_THREADS + threadIdx.x) / TK_CAP], order_key(mine_v[q]));
    __syncthreads();
    bool complete = true;
    for (int c = 0; c < TK_CHUNKS; ++c) complete = complete && (part_n[c] == 0 || least[c] < order_key(cut));
    if (!complete) return;
#pragma unroll
    for (int q = 0; q < PER; ++q)
      if (mine[q] && !(mine_v[q] < cut)) {
        const int slot = atomicAdd(&S.n, 1);
        if (slot < SAMP_CAND) {
          S.cv[slot] = mine_v[q];
          S.ci[slot] = mine_i[q];
        }
      }
    __syncthreads();
    if (S.n > SAMP_CAND) return;
  } else {
#pragma unroll
    for (int q = 0; q < PER; ++q)
      if (mine[q]) {
        const uint32_t bin = (kmax - order_key(mine_v[q])) >> 16;
        if (bin < 255u) atomicAdd(&hist[bin], 1);
        if (big_k) atomicMin(&least[(q * SAMP_THREADS + threadIdx.x) / TK_CAP], order_key(mine_v[q]));
      }
    __syncthreads();
    if (threadIdx.x < WAVE) {
      int cum, b;
      first_bin_reaching(hist, k, &b, &cum);
      if (threadIdx.x == 0) bstar = b < 255 && cum <= SAMP_CAND ? b : -1;
    }
    __syncthreads();
    if (bstar < 0) return;
    if (big_k) {
      // the parts offered their largest TK_CAP, not their largest k: everything within the cut's distance is here only
      // if each part's smallest offer lies farther from the maximum than that
      bool complete = true;
      for (int c = 0; c < TK_CHUNKS; ++c) complete = complete && (part_n[c] == 0 || ((kmax - least[c]) >> 16) > (uint32_t)bstar);
      if (!complete) return;
    }
#pragma unroll
    for (int q = 0; q < PER; ++q)
      if (mine[q] && ((kmax - order_key(mine_v[q])) >> 16) <= (uint32_t)bstar) {
        const int slot = atomicAdd(&S.n, 1);
        S.cv[slot] = mine_v[q];
        S.ci[slot] = mine_i[q];
      }
  }
  __syncthreads();
  const int pick = sample_small(S, S.n, by_min_p ? 0x7fffffff : k, top, top_p[row], min_p[row], uniform[row]);
  if (threadIdx.x == 0) {
    out[row] = pick;
    const int rr = recent_rows ? recent_rows[row] : row;
    if (counts && n_recent > 0) {
      recent[(size_t)rr * n_recent + counts[rr] % n_recent] = pick;
      counts[rr] += 1;
    }
    ((int*)scratch)[TK_DONE] = 1;
  }
}

__global__ __launch_bounds__(SAMP_THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int V,
                                                              float* __restrict__ work_all,
                                                              const float* __restrict__ temperature,
                                                              const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                              const float* __restrict__ min_p, const float* __restrict__ penalty,
                                                              int32_t* __restrict__ recent, int n_recent,
                                                              const int32_t* __restrict__ recent_rows, int32_t* __restrict__ counts,
                                                              const float* __restrict__ uniform, int32_t* __restrict__ out,
                                                              int staged) {
  __shared__ BestIdx redb[SAMP_WAVES];
  __shared__ SampleSmall S;
  __shared__ int hist[256];
  __shared__ int chosen, bstar, cut_bin, again;
  __shared__ unsigned long long cut_before;
  float* scan = S.scan;
  const int row = blockIdx.x;
  // staged: the kernels that deal a row to several blocks ran before this one and say which rows they finished
  if (staged && ((const int*)(work_all + (size_t)row * V))[TK_DONE] != 0) return;
  const float* lg = logits + (size_t)row * ld;
  const float temp = temperature[row];
  if (!(temp > 0.f)) {   // greedy row
    const BestIdx b = block_argmax(lg, V, redb, (V & 3) == 0 && (ld & 3) == 0 && ((uintptr_t)logits & 15) == 0);
    if (threadIdx.x == 0) out[row] = b.i < 0 ? 0 : b.i;
    return;
  }
  float* work = work_all + (size_t)row * V;
  const float inv_temp = temp == 1.0f ? 1.0f : 1.0f / temp;
  // temperature for all, then the repetition penalty (which comes first in the pipeline) redone for the few it touches.
  // The largest element is looked for on the way: the penalty only lowers values, so it stands unless it is one of the
  // penalised tokens itself, and then the row is searched again.
  const bool vec = (V & 3) == 0 && (ld & 3) == 0 && ((uintptr_t)logits & 15) == 0 && ((uintptr_t)work_all & 15) == 0;
  BestIdx seen = {-INFINITY, -1};
  auto look = [&](int i, float x) {
    if (x == x) seen = better(seen, BestIdx{x, i});
  };
  if (vec) {
#pragma unroll 8
    for (int i = threadIdx.x; i < V / 4; i += SAMP_THREADS) {
      float4 x = ((const float4*)lg)[i];
      if (inv_temp != 1.0f) {
        x.x *= inv_temp;
        x.y *= inv_temp;
        x.z *= inv_temp;
        x.w *= inv_temp;
      }
      ((float4*)work)[i] = x;
      look(4 * i, x.x);
      look(4 * i + 1, x.y);
      look(4 * i + 2, x.z);
      look(4 * i + 3, x.w);
    }
  } else {
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS) {
      const float x = inv_temp != 1.0f ? lg[i] * inv_temp : lg[i];
      work[i] = x;
      look(i, x);
    }
  }
  if (threadIdx.x == 0) again = 0;
  BestIdx top = block_best(seen, redb);      // (its barriers also put the row in place for the reads below)
  // repetition penalty: each distinct recent token once
  // The recent tokens of this row: row `rr` of the table, all n_recent entries (-1 where empty), or with `counts` a
  // ring that holds the last min(counts[rr], n_recent) tokens, to which the token chosen here is added at the end.
  const float pen = penalty[row];
  const int rr = recent_rows ? recent_rows[row] : row;
  const int held = counts ? (counts[rr] < n_recent ? counts[rr] : n_recent) : n_recent;
  auto finish = [&](int tok) {           // thread 0
    out[row] = tok;
    if (counts && n_recent > 0) {
      recent[(size_t)rr * n_recent + counts[rr] % n_recent] = tok;
      counts[rr] += 1;
    }
  };
  if (pen > 1.0f && n_recent > 0 && (int)threadIdx.x < held) {
    const int32_t* rc = recent + (size_t)rr * n_recent;
    const int tok = rc[threadIdx.x];
    bool first = tok >= 0 && tok < V;
    for (int j = 0; first && j < (int)threadIdx.x; ++j) first = rc[j] != tok;
    if (first) {
      const float x = lg[tok] > 0.f ? lg[tok] / pen : lg[tok] * pen;
      work[tok] = inv_temp != 1.0f ? x * inv_temp : x;
      if (tok == top.i) again = 1;
    }
  }
  __syncthreads();
  if (again) top = block_argmax(work, V, redb, vec);
  const int k = top_k[row];
  const float tp = top_p[row], mp = min_p[row];
  // top-k: everything below the k-th largest value is masked; ties at it stay
  if (k > 0 && k < V) {
    // Quick way: count the elements by their distance below the maximum (in steps of 2^16 of the ordered bit
    // pattern: a sixteenth of a unit around 10), find the distance within which k of them lie, and if those are few,
    // carry on with them alone.
    const uint32_t kmax = order_key(top.v);
    if (threadIdx.x < 256) hist[threadIdx.x] = 0;
    if (threadIdx.x == 0) {
      bstar = -1;
      S.n = 0;
    }
    __syncthreads();
    for_each_element(work, V, vec, [&](int, float x) {
      const uint32_t bin = (kmax - order_key(x)) >> 16;
      if (bin < 255u) atomicAdd(&hist[bin], 1);
    });
    __syncthreads();
    if (threadIdx.x == 0) {
      int cum = 0;
      for (int b = 0; b < 255; ++b) {
        cum += hist[b];
        if (cum >= k) {
          if (cum <= SAMP_CAND) bstar = b;
          break;
        }
      }
    }
    __syncthreads();
    if (bstar >= 0) {
      const uint32_t lim = (uint32_t)bstar;
      for_each_element(work, V, vec, [&](int i, float x) {
        if (((kmax - order_key(x)) >> 16) <= lim) {
          const int slot = atomicAdd(&S.n, 1);
          S.cv[slot] = x;
          S.ci[slot] = i;
        }
      });
      __syncthreads();
      const int pick = sample_small(S, S.n, k, top, tp, mp, uniform[row]);
      if (threadIdx.x == 0) finish(pick);
      return;
    }
    // many equal values at the cut, or the k-th value far below the maximum: the cut from counts over the whole row
    __shared__ int cut_at[2];
    const uint32_t tau = radix_threshold(work, V, k, (int*)S.sv, cut_at, vec);
    for (int i = threadIdx.x; i < V; i += SAMP_THREADS)
      if (order_key(work[i]) < tau) work[i] = -INFINITY;
    __syncthreads();
  }
  // What top-p and min-p cut is not written into the row: the draw, which is all that reads the row after them, leaves
  // out what lies below the two cuts as it goes (a pass over the row costs one compute unit 11 us and more).
  uint32_t cut_key = 0u;                 // top-p: elements whose ordered key is below this are out
  float cut_value = -INFINITY;           // min-p: elements below this are out
  // top-p: smallest set, by falling probability, whose mass reaches p
  if (tp < 1.0f) {
    // The cut is the largest value tau with mass({x >= tau}) >= p * (all the mass).  Masses are exp(x - max) in fixed
    // point (units of 2^-32) with 64-bit sums: the order of additions does not matter, so atomic additions in LDS give
    // the same cut every time.  The cut's distance below the maximum, in steps of the ordered bit pattern, is found
    // 11, 11 and 10 bits at a time, each time from a histogram of masses: three passes over the row.
    unsigned long long* hist64 = (unsigned long long*)S.sv;     // 2048 bins: sv, si, se and skey, which lie together
    unsigned long long* tmp64 = (unsigned long long*)S.cv;      // 1024 sums: cv and ci
    static_assert(offsetof(SampleSmall, skey) - offsetof(SampleSmall, sv) == 3 * SAMP_CAND * 4 && SAMP_CAND * 16 == 2048 * 8 &&
                      offsetof(SampleSmall, ci) - offsetof(SampleSmall, cv) == SAMP_CAND * 4 && SAMP_THREADS == 1024,
                  "the histogram borrows the candidates' arrays");
    const uint32_t kmax = order_key(top.v);
    uint32_t prefix = 0;            // the distance's upper bits, as far as they are known
    unsigned long long need = 0;
    for (int level = 0; level < 3; ++level) {
      const int shift = level == 0 ? 21 : (level == 1 ? 10 : 0), bits = level == 2 ? 10 : 11;
      for (int b = threadIdx.x; b < 2048; b += SAMP_THREADS) hist64[b] = 0;
      __syncthreads();
      for_each_element(work, V, vec, [&](int, float x) {
        const uint32_t dist = kmax - order_key(x);
        if (level == 0 || (dist >> (shift + bits)) == prefix) {
          const float ev = expf(x - top.v);
          if (ev > 0.f) {
            const unsigned long long m = (unsigned long long)(ev * 4294967296.0f);
            if (m) atomicAdd(&hist64[(dist >> shift) & ((1u << bits) - 1u)], m);
          }
        }
      });
      __syncthreads();
      const unsigned long long a = hist64[2 * threadIdx.x], b = hist64[2 * threadIdx.x + 1];
      tmp64[threadIdx.x] = a + b;
      __syncthreads();
      for (int o = 1; o < SAMP_THREADS; o <<= 1) {      // running sums of the pairs of bins, in order
        const unsigned long long add = (int)threadIdx.x >= o ? tmp64[threadIdx.x - o] : 0ull;
        __syncthreads();
        tmp64[threadIdx.x] += add;
        __syncthreads();
      }
      const unsigned long long incl = tmp64[threadIdx.x], excl = incl - (a + b);
      if (level == 0) {
        const unsigned long long total = tmp64[SAMP_THREADS - 1];      // at least 2^32: the maximum's own mass
        need = (unsigned long long)((double)tp * (double)total);
        need = need < 1ull ? 1ull : (need > total ? total : need);
      }
      if (excl < need && need <= excl + a) {
        cut_bin = 2 * (int)threadIdx.x;
        cut_before = excl;
      } else if (excl + a < need && need <= incl) {
        cut_bin = 2 * (int)threadIdx.x + 1;
        cut_before = excl + a;
      }
      __syncthreads();
      prefix = (prefix << bits) | (uint32_t)cut_bin;
      need -= cut_before;
      __syncthreads();
    }
    cut_key = kmax - prefix;
  }
  // min-p: probability below min_p * (largest probability) is masked
  if (mp > 0.f) cut_value = top.v + logf(mp);
  // softmax and inverse-CDF draw, cumulative sums in index order.  Each wave owns a run of the row and walks it 256
  // elements at a time (four to a lane), adding them up within the lane and then by a scan over the lanes; the waves'
  // totals, added in wave order, tell which wave holds the target, and that wave walks its run once more, with the
  // same sums, to the element.
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seg = ((V + SAMP_WAVES - 1) / SAMP_WAVES + 255) / 256 * 256;
  const int w0 = wave * seg < V ? wave * seg : V, w1 = w0 + seg < V ? w0 + seg : V;
  auto scan64 = [&](float x) {          // inclusive, lanes in order
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      const float y = __shfl_up(x, o, WAVE);
      if (lane >= o) x += y;
    }
    return x;
  };
  const bool any_cut = cut_key != 0u || cut_value > -INFINITY;
  auto four = [&](int i, float* ev) {   // exp(work - top) of elements i..i+3 of the wave's run, 0 beyond it and below the cuts
    float x[4];
    if (vec && i + 3 < w1) {
      const float4 v4 = *(const float4*)(work + i);
      x[0] = v4.x; x[1] = v4.y; x[2] = v4.z; x[3] = v4.w;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) x[c] = i + c < w1 ? work[i + c] : -INFINITY;
    }
    if (any_cut) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (order_key(x[c]) < cut_key || x[c] < cut_value) x[c] = -INFINITY;
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) ev[c] = expf(x[c] - top.v);
  };
  // The totals of the 256-element pieces are kept (where the row is not too long for that), so that the wave that
  // holds the target goes straight to the piece that reaches it instead of walking its run from the start.
  float* piece_total = S.sv;            // sv, si, se and skey lie together and are free by now: 4 * SAMP_CAND floats
  const int pieces = seg / (4 * WAVE);  // of a wave's run
  const bool keep = pieces * SAMP_WAVES <= 4 * SAMP_CAND;
  float running = 0.f;
#pragma unroll 4
  for (int b = w0; b < w1; b += 4 * WAVE) {
    float ev[4];
    four(b + 4 * lane, ev);
    const float mine = ((ev[0] + ev[1]) + ev[2]) + ev[3];
    const float total = __shfl(scan64(mine), WAVE - 1, WAVE);
    running += total;
    if (keep && lane == 0) piece_total[wave * pieces + (b - w0) / (4 * WAVE)] = total;
  }
  if (lane == 0) scan[wave] = running;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  float before = 0.f, Z = 0.f;
  for (int w = 0; w < SAMP_WAVES; ++w) {
    if (w < wave) before += scan[w];
    Z += scan[w];
  }
  const float target = uniform[row] * Z;
  // the first wave whose total reaches the target (the last one with anything in it, if rounding leaves none)
  int holder = -1, last_full = -1;
  {
    float cum = 0.f;
    for (int w = 0; w < SAMP_WAVES; ++w) {
      cum += scan[w];
      if (scan[w] > 0.f) {
        last_full = w;
        if (holder < 0 && cum >= target) holder = w;
      }
    }
    if (holder < 0) holder = last_full;
  }
  if (wave == holder) {
    float cum = before;
    int pick = -1, last = -1;
    if (keep) {
      // the first piece whose end reaches the target, by the same sums in the same order as the walk below makes them.
      // (A walk from the start could stop a piece earlier, at a lane whose sum rounds above its piece's total: a draw
      // within rounding of an edge either way.  If the piece found holds no such element after all, or none reaches
      // the target, the walk from the start decides as it always did.)
      float c = before;
      int p = 0;
      const int n_mine = (w1 - w0 + 4 * WAVE - 1) / (4 * WAVE);
      for (; p < n_mine; ++p) {
        const float t = piece_total[wave * pieces + p];
        if (c + t >= target) break;
        c += t;
      }
      if (p < n_mine) {
        float ev[4];
        const int i0 = w0 + p * 4 * WAVE + 4 * lane;
        four(i0, ev);
        const float s1 = ev[0], s2 = s1 + ev[1], s3 = s2 + ev[2], s4 = s3 + ev[3];
        const float incl = scan64(s4);
        float excl = __shfl_up(incl, 1, WAVE);
        if (lane == 0) excl = 0.f;
        const float base = c + excl;
        const float sums[4] = {s1, s2, s3, s4};
        int mine_pick = -1;
#pragma unroll
        for (int e = 3; e >= 0; --e)
          if (ev[e] > 0.f && base + sums[e] >= target) mine_pick = i0 + e;
        const unsigned long long hit = __ballot(mine_pick >= 0);
        if (hit) pick = __shfl(mine_pick, __ffsll((long long)hit) - 1, WAVE);
      }
    }
    for (int b = w0; b < w1 && pick < 0; b += 4 * WAVE) {
      float ev[4];
      const int i0 = b + 4 * lane;
      four(i0, ev);
      const float s1 = ev[0], s2 = s1 + ev[1], s3 = s2 + ev[2], s4 = s3 + ev[3];
      const float incl = scan64(s4);
      float excl = __shfl_up(incl, 1, WAVE);
      if (lane == 0) excl = 0.f;
      const float base = cum + excl;
      // this lane's first element that reaches the target, and its last one with any weight
      int mine_pick = -1, mine_last = -1;
      const float sums[4] = {s1, s2, s3, s4};
#pragma unroll
      for (int c = 3; c >= 0; --c)
        if (ev[c] > 0.f) {
          if (mine_last < 0) mine_last = i0 + c;
          if (base + sums[c] >= target) mine_pick = i0 + c;
        }
      const unsigned long long hit = __ballot(mine_pick >= 0);
      const unsigned long long any = __ballot(mine_last >= 0);
      if (any) last = __shfl(mine_last, 63 - __clzll(any), WAVE);
      if (hit) pick = __shfl(mine_pick, __ffsll((long long)hit) - 1, WAVE);
      cum += __shfl(incl, WAVE - 1, WAVE);
    }
    if (lane == 0) chosen = pick >= 0 ? pick : last;
  }
  __syncthreads();
  if (threadIdx.x == 0) finish(chosen >= 0 ? chosen : (top.i < 0 ? 0 : top.i));
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

// The first stage's candidates for dlgo_argmax_noalloc.  In host code this name is only a handle: the array's address
// on a device comes from hipGetSymbolAddress, once per device, and is what the kernels are given.
static __device__ __align__(256) unsigned char argmax_scratch[DLGO_ARGMAX_NOALLOC_ROWS * ARGMAX_CHUNKS * sizeof(BestIdx)];
#define DLGO_MAX_DEVICES 64
static void* argmax_scratch_ptr[DLGO_MAX_DEVICES];
static std::mutex argmax_scratch_lock;

// The address of the current device's copy of the array, asked of the runtime the first time it is wanted there.
static const char* argmax_scratch_here(void** where) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  DLGO_REQUIRE(e == hipSuccess, "argmax: hipGetDevice failed: %s", hipGetErrorString(e));
  DLGO_REQUIRE(dev >= 0 && dev < DLGO_MAX_DEVICES, "argmax: device %d is beyond the %d this library keeps scratch for", dev, DLGO_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(argmax_scratch_lock);
  if (!argmax_scratch_ptr[dev]) {        // this device's copy of the array, with this device current
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_scratch));
    DLGO_REQUIRE(e == hipSuccess && p, "argmax: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
    argmax_scratch_ptr[dev] = p;
  }
  *where = argmax_scratch_ptr[dev];
  return nullptr;
}

extern "C" const char* dlgo_argmax_noalloc_init() {
  void* p;
  return argmax_scratch_here(&p);
}

extern "C" const char* dlgo_argmax_noalloc(const float* logits, int ld, int n_rows, int V, int32_t* out, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
  DLGO_REQUIRE(n_rows <= DLGO_ARGMAX_NOALLOC_ROWS, "argmax without allocation: at most %d rows at a time, got %d",
               DLGO_ARGMAX_NOALLOC_ROWS, n_rows);
  DLGO_REQUIRE(logits && out, "argmax: missing argument");
  void* partial = nullptr;
  if (const char* err = argmax_scratch_here(&partial)) return err;
  if (n_rows == 0) return nullptr;
  hipLaunchKernelGGL(argmax_part_kernel, dim3(ARGMAX_CHUNKS, n_rows), dim3(ARGMAX_THREADS), 0, stream, logits, ld, V, (BestIdx*)partial);
  DLGO_LAUNCH_CHECK("argmax");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(WAVE), 0, stream, (const BestIdx*)partial, out);
  DLGO_LAUNCH_CHECK("argmax");
  return nullptr;
}

// work: [n_rows, V] float32 scratch.  dealt_rows: 1 unless the caller knows the rows' options and none is of a kind that
// several blocks share (a top-k of 1 to 1,024, or neither top-k nor top-p); a row is drawn from the same distribution either way,
// and a row with a top-k gets the same token.  recent: a table of token ids with n_recent columns.  Without counts, row r of
// it holds row r's recent tokens, -1 where empty.  With recent_rows and counts, row recent_rows[r] of it is a ring of the
// last tokens chosen for that key, counts[key] the number chosen so far; the kernel adds the token it chooses.
extern "C" const char* dlgo_sample(const float* logits, int ld, int n_rows, int V, float* work,
                                   const float* temperature, const int32_t* top_k, const float* top_p, const float* min_p,
                                   const float* penalty, int32_t* recent, int n_recent, const int32_t* recent_rows,
                                   int32_t* counts, const float* uniform, int32_t* out, int dealt_rows, hipStream_t stream) {
  DLGO_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
  DLGO_REQUIRE(n_recent >= 0 && n_recent <= SAMP_THREADS, "sample: at most %d recent tokens, got %d", SAMP_THREADS, n_recent);
  DLGO_REQUIRE(work && temperature && top_k && top_p && min_p && penalty && uniform && out, "sample: missing argument");
  DLGO_REQUIRE(n_recent == 0 || recent, "sample: recent tokens missing");
  DLGO_REQUIRE((recent_rows == nullptr) == (counts == nullptr), "sample: a ring of recent tokens needs both its rows and its counts");
  if (n_rows == 0) return nullptr;
  // a wide vocabulary: rows with a small top-k, and rows that nothing cuts, are dealt to several blocks first;
  // sample_kernel takes what they leave
  // (dealt_rows: 0 = the caller knows that no row is one the two kernels take, so they would find nothing to do)
  const int staged = dealt_rows != 0 && V >= TK_MIN_V && V <= TK_CHUNKS * TK_CHUNK_MAX && V >= TK_SCRATCH && n_rows <= 65535;
  if (staged) {
    hipLaunchKernelGGL(topk_part_kernel, dim3(TK_CHUNKS, n_rows), dim3(TK_THREADS), 0, stream, logits, ld, V, work, temperature,
                       top_k, top_p, min_p, penalty, recent, n_recent, recent_rows, counts);
    DLGO_LAUNCH_CHECK("sample (the rows' parts)");
    hipLaunchKernelGGL(topk_final_kernel, dim3(n_rows), dim3(SAMP_THREADS), 0, stream, logits, ld, V, work, temperature, top_k,
                       top_p, min_p, penalty, recent, n_recent, recent_rows, counts, uniform, out);
    DLGO_LAUNCH_CHECK("sample (the rows' cuts)");
  }
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMP_THREADS), 0, stream, logits, ld, V, work, temperature, top_k, top_p,
                     min_p, penalty, recent, n_recent, recent_rows, counts, uniform, out, staged);
  DLGO_LAUNCH_CHECK("sample");
  return nullptr;
}

#include "exact_end.h"

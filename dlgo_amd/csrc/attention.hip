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
//   attn_rows_kernel     any dtype; one wave per (token, query head), online
//                        softmax page by page in float32.  The float32 path.
//   attn_prefill_kernel  bfloat16; flash-style: a block takes 128 query rows
//                        (tokens x the heads of one group) that share one KV head,
//                        walks the pages of keys through LDS, and keeps scores
//                        transposed (keys x rows) so that each lane owns one query
//                        row: softmax statistics stay in the lane and the
//                        probabilities feed the second MFMA without a shuffle.
//   attn_decode_kernel   bfloat16; one token per sequence: the waves of a block take the
//                        pages of one (sequence, KV head), all heads of the group
//                        at once as the MFMA's 16 columns,
//                        in turn; the waves of a block are merged through LDS, and
//                        blocks, when a long sequence is split over several, by
//                        attn_combine_kernel, always in page order.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
#define PAGE 64

static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 512, "head sizes come in steps of 16, up to 512");

// true float32 from here (exact_begin.h): the kernel for any dtype and shape, exact in both
#include "exact_begin.h"
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

// The blocks a decode step gives the pages of a (sequence, kv head): the grid has `most`.  A sequence uses them all, or,
// where the grid is sized for the longest sequence the launch allows (chunk > 0), as many as give each block about
// `chunk` pages, at least `least`.  The blocks used share the sequence's pages evenly; the others return at once.
struct SplitPlan {
  int most, least, chunk;
};
__device__ __forceinline__ int splits_used(const SplitPlan& sp, int n_pages) {
  if (sp.chunk <= 0) return sp.most;
  const int by_pages = (n_pages + sp.chunk / 2) / sp.chunk;
  return by_pages < sp.least ? sp.least : (by_pages > sp.most ? sp.most : by_pages);
}

template <typename T>
__global__ __launch_bounds__(WAVE) void attn_rows_kernel(const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo,
                                                         const int32_t* __restrict__ positions,
                                                         const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ page_table, int max_pages,
                                                         const T* __restrict__ cache, long long page_stride, long long v_off,
                                                         int group, int window, float scale, int n_splits,
                                                         float* __restrict__ part) {
  constexpr int HD = HEAD_DIM;
  constexpr int E = Vec16<T>::E;
  constexpr int ND = (HD + WAVE - 1) / WAVE;
  __shared__ float qs[HD];
  __shared__ float ps[PAGE];
  const int t = blockIdx.x, h = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
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

  // with n_splits > 1 the pages of the row are dealt evenly to that many blocks (as attn_decode_kernel deals them), each
  // of which leaves (values, maximum, sum) in part[((t * heads + h) * n_splits + split) * (HD + 4)], natural exponents
  const int first_pg = lo / PAGE, last_pg = pos / PAGE;
  const int span = (last_pg - first_pg + n_splits) / n_splits;
  const int pg0 = first_pg + split * span;
  const int pg1 = pg0 + span - 1 < last_pg ? pg0 + span - 1 : last_pg;
  if (pg0 > pg1) return;
  for (int pg = pg0; pg <= pg1; ++pg) {
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
  if (n_splits > 1) {
    float* dst = part + ((size_t)(t * gridDim.y + h) * n_splits + split) * (HD + 4);
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = lane + i * WAVE;
      if (d < HD) dst[d] = acc[i];
    }
    if (lane == 0) {
      dst[HD] = m;
      dst[HD + 1] = l;
    }
    return;
  }
  T* orow = out + (size_t)t * ldo + (size_t)h * HD;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = lane + i * WAVE;
    if (d < HD) Elem<T>::store(orow + d, acc[i] * inv);
  }
}

#include "exact_end.h"

// How the partial results of several blocks are weighted when they are merged: e^x for the float32 kernels' natural
// exponents (defined among them), 2^x for the bfloat16 kernels' base-2 ones.
template <bool NATURAL> __device__ __forceinline__ float merge_weight(float x);

// ----------------------------------------------------------------------------
// bfloat16 MFMA kernels
// ----------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

__device__ __forceinline__ bf16x8_t as_bf16x8(const uint4& u) {
  union { uint4 u; bf16x8_t v; } x;
  x.u = u;
  return x.v;
}
__device__ __forceinline__ bf16x8_t join_bf16x8(const uint2& lo, const uint2& hi) {
  union { uint2 u[2]; bf16x8_t v; } x;
  x.u[0] = lo;
  x.u[1] = hi;
  return x.v;
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
template <> __device__ __forceinline__ float merge_weight<false>(float x) { return fast_exp2(x); }

#define PF_THREADS 256   // threads of a team
#define PF_ROWS 128      // query rows (token x head of the group) per block
// two teams for head sizes up to 64: there a wave gets by with the 128 registers that 16 waves on a compute unit leave it
#define PF_TEAMS (HEAD_DIM <= 64 ? 2 : 1)

// Prefill.  grid (q tiles, sequences, kv heads).  bq = tokens per block (bq * group <= 128).
// (At least two waves on a SIMD leave a wave at most 256 registers, all of them ordinary ones: the compiler then keeps
// the MFMA results where the vector unit can reach them, instead of copying scores and sums in and out of the
// accumulation registers in every turn.)
__global__ __launch_bounds__(PF_THREADS* PF_TEAMS) __attribute__((amdgpu_waves_per_eu(PF_TEAMS == 2 ? 4 : 2))) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ start_pos, const int32_t* __restrict__ slots, const int32_t* __restrict__ page_table,
    int max_pages, const bf16_t* __restrict__ cache, long long page_stride, long long v_off, int group, int bq, int window,
    float scale_log2e) {
  constexpr int HD = HEAD_DIM;
  constexpr int KS = HD / 16;               // k steps of K Q^T (32x32x16)
  constexpr int DT = (HD + 31) / 32;        // 32-row tiles of the output's head dimension
  constexpr int KROW = HD * 2 + 16;         // bytes of a key row in LDS (padded)
  constexpr int VROW = PAGE * 2 + 8;        // bytes of a row of transposed values in LDS: 34 words, so that the 32 rows
                                            // that half a wave reads 8 bytes of at a time fall on different banks
  constexpr int KCH = PAGE * HD / 8;        // 16-byte chunks of a key tile
  constexpr int VCH = HD * PAGE / 8;
  constexpr int NKC = (KCH + PF_THREADS - 1) / PF_THREADS;
  constexpr int NVC = (VCH + PF_THREADS - 1) / PF_THREADS;
  constexpr int KBYTES = PAGE * KROW, VBYTES = DT * 32 * VROW;
  constexpr int TEAMS = PF_TEAMS;
  // Each team of four waves has a page of its own in LDS.  With two teams the block's pages go to them in turn, both
  // teams work on the same 128 query rows, and team 1 hands its sums to team 0 through LDS at the end.
  __shared__ __attribute__((aligned(16))) char lds_all[TEAMS * (KBYTES + VBYTES)];
  static_assert(TEAMS == 1 || TEAMS * (KBYTES + VBYTES) >= PF_ROWS * (HD + 4) * 4, "the teams' merge must fit their pages");
  char* ldsK = lds_all + (threadIdx.x / PF_THREADS) * (KBYTES + VBYTES);
  char* ldsV = ldsK + KBYTES;

  const int seq = blockIdx.y, kvh = blockIdx.z;
  const int q0 = cu_q[seq], qn = cu_q[seq + 1] - q0;
  // Late tiles see more keys than early ones.  Blocks are handed to the compute units in the order of their linear
  // index, 256 at a time: odd rounds walk the tiles forwards and even rounds backwards, so that the blocks that share
  // a unit add up to about the same number of pages.  The direction is that of the round in which the row of tiles
  // (one sequence, one kv head) starts: the same for all its blocks, so that every tile is taken exactly once.
  const int linear0 = gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const int tile = (linear0 >> 8) & 1 ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
  const int t0 = tile * bq;
  if (t0 >= qn) return;
  const int t1 = t0 + bq < qn ? t0 + bq : qn;           // tokens [t0, t1) of the sequence's rows
  const int start = start_pos[seq];
  const int slot = slots[seq];
  const int kv_len = start + qn;                          // keys the cache holds for this sequence now
  const int team = threadIdx.x / PF_THREADS;
  const int tid = threadIdx.x % PF_THREADS, lane = tid & 63, wave = tid >> 6, half = lane >> 5;     // within the team

  // this lane's query row
  const int r = wave * 32 + (lane & 31);
  const int tok = t0 + r / group, hig = r % group;
  const bool row_ok = tok < t1;
  const int pos = row_ok ? start + tok : -1;
  const int lo = (row_ok && window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // the wave's rows span tokens [wt0, wt1]
  const int wt0 = t0 + (wave * 32) / group;
  int wt1 = t0 + (wave * 32 + 31) / group;
  wt1 = wt1 < t1 - 1 ? wt1 : t1 - 1;
  const bool wave_ok = wt0 < t1;
  const int w_pos_min = start + wt0, w_pos_max = start + wt1;
  const int w_lo_max = window > 0 && w_pos_max - window + 1 > 0 ? w_pos_max - window + 1 : 0;
  const int w_lo_min = window > 0 && w_pos_min - window + 1 > 0 ? w_pos_min - window + 1 : 0;

  uint4 qf[KS];
  {
    const bf16_t* qrow = q + (size_t)(q0 + (row_ok ? tok : t0)) * ldq + (size_t)(kvh * group + hig) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_ok ? *(const uint4*)(qrow + ks * 16 + half * 8) : make_uint4(0, 0, 0, 0);
  }
  f32x16_t o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[d][v] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int b_lo = window > 0 && start + t0 - window + 1 > 0 ? start + t0 - window + 1 : 0;
  const int pg_lo = b_lo / PAGE, pg_hi = (start + t1 - 1) / PAGE;

  uint4 rk[NKC], rv[NVC];
  auto fetch = [&](int pg) {
    const int page = page_table[(size_t)slot * max_pages + pg];
    const bf16_t* kpage = cache + (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * PAGE * HD;
    const bf16_t* vpage = cache + v_off + (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * HD * PAGE;
#pragma unroll
    for (int i = 0; i < NKC; ++i) {
      const int c = tid + i * PF_THREADS;
      rk[i] = c < KCH ? *(const uint4*)(kpage + (size_t)c * 8) : make_uint4(0, 0, 0, 0);
    }
    const bool tail = pg * PAGE + PAGE > kv_len;      // keys beyond the sequence: their values must not reach the product
#pragma unroll
    for (int i = 0; i < NVC; ++i) {
      const int c = tid + i * PF_THREADS;
      uint4 u = c < VCH ? *(const uint4*)(vpage + (size_t)c * 8) : make_uint4(0, 0, 0, 0);
      if (tail) {
        const int k0 = pg * PAGE + (c & 7) * 8;
        uint32_t* w = (uint32_t*)&u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (k0 + 2 * e >= kv_len) w[e] = 0;
          else if (k0 + 2 * e + 1 >= kv_len) w[e] &= 0xffffu;
        }
      }
      rv[i] = u;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < NKC; ++i) {
      const int c = tid + i * PF_THREADS;
      if (c < KCH) *(uint4*)(ldsK + (c / (HD / 8)) * KROW + (c % (HD / 8)) * 16) = rk[i];
    }
#pragma unroll
    for (int i = 0; i < NVC; ++i) {
      const int c = tid + i * PF_THREADS;
      if (c < VCH) {                          // rows are 8-byte aligned only
        *(uint2*)(ldsV + (c >> 3) * VROW + (c & 7) * 16) = make_uint2(rv[i].x, rv[i].y);
        *(uint2*)(ldsV + (c >> 3) * VROW + (c & 7) * 16 + 8) = make_uint2(rv[i].z, rv[i].w);
      }
    }
  };

  // turn n: team t takes page pg_lo + n * TEAMS + t, if the block has that many
  const int turns = (pg_hi - pg_lo + TEAMS) / TEAMS;
  if (pg_lo + team <= pg_hi) fetch(pg_lo + team);
  for (int turn = 0; turn < turns; ++turn) {
    const int pg = pg_lo + turn * TEAMS + team;
    const bool mine = pg <= pg_hi;
    if (mine) stash();
    __syncthreads();
    if (pg + TEAMS <= pg_hi) fetch(pg + TEAMS);
    const int key0 = pg * PAGE;
    if (mine && wave_ok && key0 <= w_pos_max && key0 + PAGE - 1 >= w_lo_min) {
      f32x16_t s[2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[kt][v] = 0.f;
        const char* pk = ldsK + (kt * 32 + (lane & 31)) * KROW + half * 16;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(*(const uint4*)(pk + ks * 32)), as_bf16x8(qf[ks]), s[kt], 0, 0, 0);
      }
      // lane: row = lane%32; element v of tile kt is key  key0 + 32 kt + 8 (v/4) + 4 half + v%4
      // m is the running maximum of the raw scores; the scale (times log2 e) enters with the exponent, one fused
      // multiply-add a score
      const bool need_mask = key0 + PAGE - 1 > w_pos_min || key0 < w_lo_max;
      float mx = -INFINITY;
      if (need_mask) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + kt * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
            s[kt][v] = (key <= pos && key >= lo) ? s[kt][v] : -INFINITY;
          }
      }
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[kt][v]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      const float m_new = fmaxf(m, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float off = -m_use * scale_log2e;
      float rs = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = fast_exp2(fmaf(s[kt][v], scale_log2e, off));
          s[kt][v] = p;
          rs += p;
        }
      rs += __shfl_xor(rs, 32, WAVE);
      if (__any(m_new != m)) {               // the sums so far are rescaled only when some row's maximum moved
        const float alpha = fast_exp2(fmaf(m, scale_log2e, off));
        l *= alpha;
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[d][v] *= alpha;
      }
      l += rs;
      m = m_new;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          bf16x8_t pb;
#pragma unroll
          for (int e = 0; e < 8; ++e) pb[e] = (__bf16)s[kt][8 * u + e];
          // element e of this operand is key 32 kt + 16 u + 8 (e/4) + 4 half + e%4: the values follow the same order
          const char* pv = ldsV + (lane & 31) * VROW + (kt * 32 + 16 * u + 4 * half) * 2;
#pragma unroll
          for (int d = 0; d < DT; ++d) {
            const uint2 lo8 = *(const uint2*)(pv + d * 32 * VROW);
            const uint2 hi8 = *(const uint2*)(pv + d * 32 * VROW + 16);
            o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(join_bf16x8(lo8, hi8), pb, o[d], 0, 0, 0);
          }
        }
    }
    __syncthreads();
  }
  if (TEAMS == 2) {
    // team 1 leaves, for each of its rows, the weighted values, the maximum and the sum; team 0 adds them to its own
    float* mrg = (float*)lds_all + (size_t)r * (HD + 4);      // rows of 16-byte pieces
    if (team == 1) {
#pragma unroll
      for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const int dd = d * 32 + 8 * qd + 4 * half;
          if (dd < HD) *(float4*)(mrg + dd) = make_float4(o[d][4 * qd], o[d][4 * qd + 1], o[d][4 * qd + 2], o[d][4 * qd + 3]);
        }
      if (half == 0) {
        mrg[HD] = m;
        mrg[HD + 1] = l;
      }
    }
    __syncthreads();
    if (team == 1) return;
    const float m2 = mrg[HD], l2 = mrg[HD + 1];
    const float mm = fmaxf(m, m2);
    const float m_use = mm == -INFINITY ? 0.f : mm;
    const float a1 = fast_exp2((m - m_use) * scale_log2e), a2 = fast_exp2((m2 - m_use) * scale_log2e);
    l = l * a1 + l2 * a2;
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int dd = d * 32 + 8 * qd + 4 * half;
        if (dd < HD) {
          const float4 o2 = *(const float4*)(mrg + dd);
          o[d][4 * qd] = o[d][4 * qd] * a1 + o2.x * a2;
          o[d][4 * qd + 1] = o[d][4 * qd + 1] * a1 + o2.y * a2;
          o[d][4 * qd + 2] = o[d][4 * qd + 2] * a1 + o2.z * a2;
          o[d][4 * qd + 3] = o[d][4 * qd + 3] * a1 + o2.w * a2;
        }
      }
  }
  if (!row_ok) return;
  const float inv = 1.0f / l;
  bf16_t* orow = out + (size_t)(q0 + tok) * ldo + (size_t)(kvh * group + hig) * HD;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int dd = d * 32 + 8 * qd + 4 * half;
      if (dd < HD) {
        uint2 pk;
        pk.x = (uint32_t)f32_to_bf16(o[d][4 * qd] * inv) | ((uint32_t)f32_to_bf16(o[d][4 * qd + 1] * inv) << 16);
        pk.y = (uint32_t)f32_to_bf16(o[d][4 * qd + 2] * inv) | ((uint32_t)f32_to_bf16(o[d][4 * qd + 3] * inv) << 16);
        *(uint2*)(orow + dd) = pk;
      }
    }
}

// Prefill in float32, for head sizes up to 128: a thread owns a query row (token x head of the group, 128 rows a block),
// a page of keys and of transposed values sits in LDS, and every product is an FMA on float32 with exact expf; the
// keys are taken 16 at a time so that the scores stay in registers.  grid and bq as attn_prefill_kernel.
#include "exact_begin.h"      // the float32 prompt kernel: true float32
template <> __device__ __forceinline__ float merge_weight<true>(float x) { return expf(x); }
#if HEAD_DIM <= 128
#define PF32_THREADS 128
__global__ __launch_bounds__(PF32_THREADS) void attn_prefill_f32_kernel(
    const float* __restrict__ q, int ldq, float* __restrict__ out, int ldo, const int32_t* __restrict__ cu_q,
    const int32_t* __restrict__ start_pos, const int32_t* __restrict__ slots, const int32_t* __restrict__ page_table,
    int max_pages, const float* __restrict__ cache, long long page_stride, long long v_off, int group, int bq, int window,
    float scale) {
  constexpr int HD = HEAD_DIM;
  constexpr int CH = PAGE * HD / 4;                 // 16-byte chunks of a page of keys (and of values)
  __shared__ __attribute__((aligned(16))) float ldsK[PAGE * HD];
  __shared__ __attribute__((aligned(16))) float ldsV[HD * PAGE];
  const int seq = blockIdx.y, kvh = blockIdx.z;
  const int q0 = cu_q[seq], qn = cu_q[seq + 1] - q0;
  const int linear0 = gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const int tile = (linear0 >> 8) & 1 ? blockIdx.x : gridDim.x - 1 - blockIdx.x;     // as attn_prefill_kernel
  const int t0 = tile * bq;
  if (t0 >= qn) return;
  const int t1 = t0 + bq < qn ? t0 + bq : qn;
  const int start = start_pos[seq], slot = slots[seq];
  const int kv_len = start + qn;
  const int tid = threadIdx.x;
  const int tok = t0 + tid / group, hig = tid % group;
  const bool row_ok = tid < bq * group && tok < t1;
  const int pos = row_ok ? start + tok : -1;
  const int lo = (row_ok && window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  float qr[HD], o[HD];
  {
    const float* qrow = q + (size_t)(q0 + (row_ok ? tok : t0)) * ldq + (size_t)(kvh * group + hig) * HD;
#pragma unroll
    for (int d = 0; d < HD; d += 4) {
      const float4 v = *(const float4*)(qrow + d);
      qr[d] = v.x * scale;
      qr[d + 1] = v.y * scale;
      qr[d + 2] = v.z * scale;
      qr[d + 3] = v.w * scale;
    }
  }
#pragma unroll
  for (int d = 0; d < HD; ++d) o[d] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int b_lo = window > 0 && start + t0 - window + 1 > 0 ? start + t0 - window + 1 : 0;
  const int pg_lo = b_lo / PAGE, pg_hi = (start + t1 - 1) / PAGE;
  for (int pg = pg_lo; pg <= pg_hi; ++pg) {
    const int page = page_table[(size_t)slot * max_pages + pg];
    const float* kpage = cache + (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * PAGE * HD;
    const float* vpage = cache + v_off + (size_t)(page < 0 ? 0 : page) * page_stride + (size_t)kvh * HD * PAGE;
    const int key0 = pg * PAGE;
    __syncthreads();                                  // the page before is done with
    for (int c = tid; c < CH; c += PF32_THREADS) {
      ((float4*)ldsK)[c] = ((const float4*)kpage)[c];
      float4 v = ((const float4*)vpage)[c];
      const int k = key0 + (c % (PAGE / 4)) * 4;      // values of keys beyond the sequence must not reach the sums
      if (k >= kv_len) v.x = 0.f;
      if (k + 1 >= kv_len) v.y = 0.f;
      if (k + 2 >= kv_len) v.z = 0.f;
      if (k + 3 >= kv_len) v.w = 0.f;
      ((float4*)ldsV)[c] = v;
    }
    __syncthreads();
    if (!row_ok || key0 > pos || key0 + PAGE - 1 < lo) continue;
    for (int g = 0; g < PAGE / 16; ++g) {
      const int kbase = key0 + 16 * g;
      if (kbase > pos || kbase + 15 < lo) continue;
      float s[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const float* kr = ldsK + (16 * g + k) * HD;
        float a = 0.f;
#pragma unroll
        for (int d = 0; d < HD; d += 4) {
          const float4 kv = *(const float4*)(kr + d);
          a = fmaf(qr[d], kv.x, a);
          a = fmaf(qr[d + 1], kv.y, a);
          a = fmaf(qr[d + 2], kv.z, a);
          a = fmaf(qr[d + 3], kv.w, a);
        }
        const int key = kbase + k;
        s[k] = (key <= pos && key >= lo) ? a : -INFINITY;
      }
      float mx = s[0];
#pragma unroll
      for (int k = 1; k < 16; ++k) mx = fmaxf(mx, s[k]);
      const float m_new = fmaxf(m, mx);               // finite: the group holds a key this row sees
      const float alpha = expf(m - m_new);            // 0 the first time (m = -inf)
      float rs = 0.f;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        s[k] = expf(s[k] - m_new);
        rs += s[k];
      }
      l = l * alpha + rs;
      m = m_new;
#pragma unroll
      for (int d = 0; d < HD; ++d) {
        const float* vr = ldsV + d * PAGE + 16 * g;
        float a = o[d] * alpha;
#pragma unroll
        for (int k = 0; k < 16; k += 4) {
          const float4 vv = *(const float4*)(vr + k);
          a = fmaf(s[k], vv.x, a);
          a = fmaf(s[k + 1], vv.y, a);
          a = fmaf(s[k + 2], vv.z, a);
          a = fmaf(s[k + 3], vv.w, a);
        }
        o[d] = a;
      }
    }
  }
  if (!row_ok) return;
  const float inv = 1.0f / l;
  float* orow = out + (size_t)(q0 + tok) * ldo + (size_t)(kvh * group + hig) * HD;
#pragma unroll
  for (int d = 0; d < HD; d += 4) *(float4*)(orow + d) = make_float4(o[d] * inv, o[d + 1] * inv, o[d + 2] * inv, o[d + 3] * inv);
}
#endif
#include "exact_end.h"

// Rotation of 8 consecutive elements d0..d0+7 of one head vector (bfloat16) at a position whose cos/sin rows are
// given, as rope_kv.hip does it: split-half pairs (d, d + rot/2) or interleaved pairs (2i, 2i+1); elements from
// `rot` on are copied.  rot is a multiple of 16, so the 8 elements lie in one half.
__device__ __forceinline__ uint4 rotated8(const bf16_t* __restrict__ vec, int d0, const float* __restrict__ cs,
                                          const float* __restrict__ sn, int rot, int interleaved) {
  const uint4 raw = *(const uint4*)(vec + d0);
  if (cs == nullptr || d0 >= rot) return raw;
  float x[8], y[8];
  Vec16<bf16_t>::load(vec + d0, x);
  if (interleaved) {
    const float4 c4 = *(const float4*)(cs + d0 / 2), s4 = *(const float4*)(sn + d0 / 2);
    const float c[4] = {c4.x, c4.y, c4.z, c4.w}, sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y[2 * i] = rotated_lo(x[2 * i], x[2 * i + 1], c[i], sv[i]);
      y[2 * i + 1] = rotated_hi(x[2 * i], x[2 * i + 1], c[i], sv[i]);
    }
  } else {
    const int half = rot / 2;
    const bool low = d0 < half;
    const int i0 = low ? d0 : d0 - half;
    float p[8], c[8], sv[8];
    Vec16<bf16_t>::load(vec + (low ? d0 + half : d0 - half), p);
    *(float4*)c = *(const float4*)(cs + i0);
    *(float4*)(c + 4) = *(const float4*)(cs + i0 + 4);
    *(float4*)sv = *(const float4*)(sn + i0);
    *(float4*)(sv + 4) = *(const float4*)(sn + i0 + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = low ? rotated_lo(x[e], p[e], c[e], sv[e]) : rotated_hi(p[e], x[e], c[e], sv[e]);
  }
  union { uint4 u; bf16x8_t v; } o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o.v[e] = (__bf16)y[e];
  return o.u;
}

// Decode: one token per sequence.  grid (splits, kv heads x head blocks of 16, sequences), NWV waves per block.
// The pages that hold keys of a sequence's token are dealt evenly to the splits; a block's waves take its pages
// in turn (wave w: the first page + w, + NWV, ...), all heads of the group at once as the MFMA's 16 columns, and are merged
// through LDS in wave order.  With one split the block writes the finished rows; else it writes a partial per
// head, part[((seq * H + head) * n_splits + split) * (HD + 4)] = weighted values [HD], max, sum (base-2
// exponents), 2 unused, and attn_combine_kernel merges the partials in page order.
//
// With cos/sin tables given, q holds the step's unrotated rows [q | k | v]: the query heads are rotated as they are
// read, and (new_kv) the token's own key and value are taken from the row instead of the cache: the wave that
// holds the token's page rotates the key, puts key and value into its operands and writes them to the cache for
// the steps to come (rope_kv.hip's work, without its launch).
template <int NWV, bool FUSED>
__global__ __launch_bounds__(NWV* WAVE) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, float* __restrict__ part,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, const int32_t* __restrict__ page_table,
    int max_pages, bf16_t* __restrict__ cache, long long page_stride, long long v_off, int n_heads, int group,
    int head_blocks, SplitPlan sp, int window, float scale_log2e, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rot, int interleaved, int new_kv, int k_col, int v_col) {
  constexpr int HD = HEAD_DIM;
  constexpr int KS = (HD + 31) / 32;   // k steps of K Q^T (16x16x32)
  constexpr int DT = HD / 16;          // 16-row tiles of the output's head dimension
  constexpr int LS = HD + 2;           // floats a wave leaves in LDS per head: values, max, sum
  extern __shared__ float lds[];
  // the split is the slowest index: the blocks of a short sequence that have pages are then neighbours in launch order,
  // which is dealt round to the XCDs, and not every fourth or eighth block on the same few of them
  const int split = blockIdx.z, seq = blockIdx.y;
  const int kvh = blockIdx.x / head_blocks, hb = blockIdx.x % head_blocks;
  const int pos = positions[seq];
  const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
  // the pages that hold keys of this token are dealt evenly to the splits
  const int first_pg = lo / PAGE, last_pg = pos / PAGE;
  const int n_splits = sp.most, used = splits_used(sp, last_pg - first_pg + 1);
  const int span = (last_pg - first_pg + used) / used;
  const int pg0 = first_pg + split * span;
  const int pg1 = pg0 + span - 1 < last_pg ? pg0 + span - 1 : last_pg;
  if (pg0 > pg1) return;               // the whole block: fewer pages than splits
  const int slot = slots[seq];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = lane & 15, G = lane >> 4;
  const int hig = hb * 16 + j;                    // head within the group
  const int heads_here = group - hb * 16 < 16 ? group - hb * 16 : 16;
  const bool head_ok = j < heads_here;
  const int head = kvh * group + hig;

  const float* cs = cos_t ? cos_t + (size_t)pos * (rot / 2) : nullptr;
  const float* sn = cos_t ? sin_t + (size_t)pos * (rot / 2) : nullptr;
  uint4 qf[KS];
  bool have_q = false;                 // the queries are read (and rotated) behind the first page's loads
  f32x4_t o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int own = pos % PAGE;          // the token's own row in its page

  for (int pg = pg0 + wave; pg <= pg1; pg += NWV) {
    const int page = page_table[(size_t)slot * max_pages + pg];
    if (page < 0) continue;
    bf16_t* kpage = cache + (size_t)page * page_stride + (size_t)kvh * PAGE * HD;
    bf16_t* vpage = cache + v_off + (size_t)page * page_stride + (size_t)kvh * HD * PAGE;
    const int key0 = pg * PAGE;
    // every load of the page is issued before the first product
    uint4 kf[4][KS];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16_t* krow = kpage + (size_t)(t * 16 + j) * HD + G * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[t][ks] = (ks * 32 + G * 8 < HD) ? *(const uint4*)(krow + ks * 32) : make_uint4(0, 0, 0, 0);
    }
    uint2 vf[2][DT][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const bf16_t* vrow = vpage + (size_t)(d * 16 + j) * PAGE + 32 * u + 4 * G;
        vf[u][d][0] = *(const uint2*)(vrow);
        vf[u][d][1] = *(const uint2*)(vrow + 16);
      }
    if (!have_q) {
      have_q = true;
      const bf16_t* qrow = q + (size_t)seq * ldq + (size_t)(head_ok ? head : kvh * group) * HD;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[ks] = !(head_ok && ks * 32 + G * 8 < HD) ? make_uint4(0, 0, 0, 0)
                 : (FUSED ? rotated8(qrow, ks * 32 + G * 8, cs, sn, rot, interleaved) : *(const uint4*)(qrow + ks * 32 + G * 8));
    }
    if (FUSED && new_kv && pg == last_pg) {
      // the token's own key and value come from the step's row, not from the cache; head block 0 stores them
      const bf16_t* row = q + (size_t)seq * ldq;
      const bf16_t* krow_new = row + k_col + (size_t)kvh * HD;
      const bf16_t* vrow_new = row + v_col + (size_t)kvh * HD;
      if (j == own % 16) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (t == own / 16) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
              if (ks * 32 + G * 8 < HD) {
                kf[t][ks] = rotated8(krow_new, ks * 32 + G * 8, cs, sn, rot, interleaved);
                if (hb == 0) *(uint4*)(kpage + (size_t)own * HD + ks * 32 + G * 8) = kf[t][ks];
              }
          }
      }
      const int rr = own % 32;
      if (G == (rr % 16) / 4) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
          if (u == own / 32) {
#pragma unroll
            for (int d = 0; d < DT; ++d) {
              const bf16_t val = vrow_new[d * 16 + j];
              const int e = rr % 4;
#pragma unroll
              for (int h = 0; h < 2; ++h)
                if (h == rr / 16) {
                  uint32_t lo32 = vf[u][d][h].x, hi32 = vf[u][d][h].y;
                  if (e == 0) lo32 = (lo32 & 0xffff0000u) | val;
                  else if (e == 1) lo32 = (lo32 & 0x0000ffffu) | ((uint32_t)val << 16);
                  else if (e == 2) hi32 = (hi32 & 0xffff0000u) | val;
                  else hi32 = (hi32 & 0x0000ffffu) | ((uint32_t)val << 16);
                  vf[u][d][h] = make_uint2(lo32, hi32);
                }
              if (hb == 0) vpage[(size_t)(d * 16 + j) * PAGE + own] = val;
            }
          }
      }
    }
    f32x4_t s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      s[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[t][ks]), as_bf16x8(qf[ks]), s[t], 0, 0, 0);
    }
    // lane: head = lane%16; element v of tile t is key  key0 + 16 t + 4 G + v
    const bool need_mask = key0 + PAGE - 1 > pos || key0 < lo;
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float sv = s[t][v] * scale_log2e;
        if (need_mask) {
          const int key = key0 + 16 * t + 4 * G + v;
          sv = (key <= pos && key >= lo) ? sv : -INFINITY;
        }
        s[t][v] = sv;
        mx = fmaxf(mx, sv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m, mx);      // finite: every page of the range holds a valid key
    const float alpha = fast_exp2(m - m_new);
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float p = fast_exp2(s[t][v] - m_new);
        s[t][v] = p;
        rs += p;
      }
    rs += __shfl_xor(rs, 16, WAVE);
    rs += __shfl_xor(rs, 32, WAVE);
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] *= alpha;
    const bool tail = key0 + PAGE - 1 > pos;   // keys beyond the sequence: their values must not reach the product
#pragma unroll
    for (int u = 0; u < 2; ++u) {              // 32 keys each: tiles 2u and 2u+1
      bf16x8_t pb;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pb[e] = (__bf16)s[2 * u][e];
        pb[4 + e] = (__bf16)s[2 * u + 1][e];
      }
      const int ka = 32 * u + 4 * G, kb = ka + 16;      // first keys (within the page) of the two 4-key pieces
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        uint2 a0 = vf[u][d][0], a1 = vf[u][d][1];
        if (tail) {
          uint32_t* w0 = (uint32_t*)&a0;
          uint32_t* w1 = (uint32_t*)&a1;
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            if (key0 + ka + 2 * e > pos) w0[e] = 0;
            else if (key0 + ka + 2 * e + 1 > pos) w0[e] &= 0xffffu;
            if (key0 + kb + 2 * e > pos) w1[e] = 0;
            else if (key0 + kb + 2 * e + 1 > pos) w1[e] &= 0xffffu;
          }
        }
        o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(join_bf16x8(a0, a1), pb, o[d], 0, 0, 0);
      }
    }
  }
  // each wave leaves (values, max, sum) per head in LDS; a wave that saw no page leaves (0, -inf, 0)
  if (head_ok) {
    float* dst = lds + (size_t)(wave * heads_here + j) * LS;
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[d * 16 + 4 * G + v] = o[d][v];
    if (G == 0) {
      dst[HD] = m;
      dst[HD + 1] = l;
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < heads_here * HD; idx += NWV * WAVE) {
    const int hh = idx / HD, d = idx - hh * HD;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NWV; ++w) M = fmaxf(M, lds[(size_t)(w * heads_here + hh) * LS + HD]);
    float L = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float* src = lds + (size_t)(w * heads_here + hh) * LS;
      const float wt = fast_exp2(src[HD] - M);
      L = fmaf(wt, src[HD + 1], L);
      acc = fmaf(wt, src[d], acc);
    }
    const int hd_ = kvh * group + hb * 16 + hh;
    if (n_splits == 1) {
      out[(size_t)seq * ldo + (size_t)hd_ * HD + d] = f32_to_bf16(acc / L);
    } else {
      float* dst = part + ((size_t)(seq * n_heads + hd_) * n_splits + split) * (HD + 4);
      dst[d] = acc;
      if (d == 0) {
        dst[HD] = M;
        dst[HD + 1] = L;
      }
    }
  }
}

// The same step with the pages going through LDS.  attn_decode_kernel reads a page's keys as 16 rows x 64 bytes per
// instruction and its values in 8-byte pieces, which is what the MFMA operands look like; memory gives whole 1 KB runs
// 15 to 20% faster.  Here a wave copies its page, keys and values, into its own part of LDS with global_load_lds_dwordx4
// (1 KB of memory in a row per instruction, no registers in between), reads the operands back from there, and asks for its
// next page as soon as it holds them: the next page streams in while this one is multiplied.  A row's 16-byte
// pieces sit in LDS at slot (piece ^ f(row)), which spreads the rows a quarter wave reads at once over the banks; the
// lane that fills a slot fetches the piece that belongs there.  The keys of a page are dealt to the rows of the score
// tiles so that the eight scores a lane ends up with belong to eight consecutive tokens (tile 2u and 2u+1, rows 4G..4G+3:
// tokens 32u + 8G ..+7); the value operand of a lane is then one 16-byte piece.  Everything after the scores, the merge
// of the waves and the partial results are attn_decode_kernel's.
template <int SLOTS> struct SlotSwizzle {
  // rows whose slots share banks get different slots: the low bits of (row >> SHIFT) are XORed into the piece number, as
  // many bits as the number of pieces of a row has factors of two (at most four: sixteen 16-byte slots span the banks)
  static constexpr int P2 = (SLOTS & -SLOTS) > 16 ? 16 : (SLOTS & -SLOTS);
  static constexpr int MASK = P2 - 1;
  static constexpr int SHIFT = P2 >= 16 ? 0 : (P2 == 8 ? 1 : (P2 == 4 ? 2 : (P2 == 2 ? 3 : 0)));
  static __device__ __forceinline__ int of(int row) { return (row >> SHIFT) & MASK; }
};

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ uint4 lds_read16(const __attribute__((address_space(3))) char* p) {
  const u32x4_t v = *(const __attribute__((address_space(3))) u32x4_t*)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
static __device__ __forceinline__ void page_to_lds(const void* base, uint32_t voff, uint32_t lds_base) {
  // 16 bytes per lane from base + voff to LDS at lds_base + lane * 16 (lds_base travels in M0, the same for the wave)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(base) : "memory");
}

// what rotated8 reads, separated from what it computes, so that the loads can stand in front of a page's loads
struct Rot8In {
  uint4 x, p = {};
  float4 c0 = {}, c1 = {}, s0 = {}, s1 = {};
};
__device__ __forceinline__ Rot8In rot8_load(const bf16_t* __restrict__ vec, int d0, const float* __restrict__ cs,
                                            const float* __restrict__ sn, int rot, int interleaved) {
  // Every load is made whatever the piece needs, from a place that can be read (the piece itself where nothing is
  // wanted): with the loads under conditions the compiler waits for each before it goes on to the next, which made
  // the queries four trips to memory instead of one.
  Rot8In r;
  const bool turn = cs != nullptr && d0 < rot;
  const int half = rot / 2;
  const bool low = d0 < half;
  const bool halves = turn && !interleaved;
  const int partner = halves ? (low ? d0 + half : d0 - half) : d0;
  const int i0 = !turn ? 0 : (interleaved ? d0 / 2 : (low ? d0 : d0 - half));
  const int i1 = halves ? i0 + 4 : i0;
  const float* c = turn ? cs : (const float*)vec;
  const float* sp = turn ? sn : (const float*)vec;
  r.x = *(const uint4*)(vec + d0);
  r.p = *(const uint4*)(vec + partner);
  r.c0 = *(const float4*)(c + i0);
  r.s0 = *(const float4*)(sp + i0);
  r.c1 = *(const float4*)(c + i1);
  r.s1 = *(const float4*)(sp + i1);
  return r;
}
__device__ __forceinline__ void unpack8(const uint4& u, float* f) {
  f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
  f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
  f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
  f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ uint4 rot8_apply(const Rot8In& r, int d0, bool rotate, int rot, int interleaved) {
  if (!rotate || d0 >= rot) return r.x;
  float x[8], y[8];
  unpack8(r.x, x);
  if (interleaved) {
    const float c[4] = {r.c0.x, r.c0.y, r.c0.z, r.c0.w}, sv[4] = {r.s0.x, r.s0.y, r.s0.z, r.s0.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y[2 * i] = rotated_lo(x[2 * i], x[2 * i + 1], c[i], sv[i]);
      y[2 * i + 1] = rotated_hi(x[2 * i], x[2 * i + 1], c[i], sv[i]);
    }
  } else {
    const bool low = d0 < rot / 2;
    float p[8];
    unpack8(r.p, p);
    const float c[8] = {r.c0.x, r.c0.y, r.c0.z, r.c0.w, r.c1.x, r.c1.y, r.c1.z, r.c1.w};
    const float sv[8] = {r.s0.x, r.s0.y, r.s0.z, r.s0.w, r.s1.x, r.s1.y, r.s1.z, r.s1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = low ? rotated_lo(x[e], p[e], c[e], sv[e]) : rotated_hi(p[e], x[e], c[e], sv[e]);
  }
  union { uint4 u; bf16x8_t v; } o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o.v[e] = (__bf16)y[e];
  return o.u;
}

template <int NWV, bool FUSED>
__global__ __launch_bounds__(NWV* WAVE) void attn_decode_lds_kernel(
    const bf16_t* __restrict__ q, int ldq, bf16_t* __restrict__ out, int ldo, float* __restrict__ part,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, const int32_t* __restrict__ page_table,
    int max_pages, bf16_t* __restrict__ cache, long long page_stride, long long v_off, int n_heads, int group,
    int head_blocks, SplitPlan sp, int window, float scale_log2e, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rot, int interleaved, int new_kv, int k_col, int v_col,
    const int32_t* __restrict__ seq_pages) {
  // seq_pages (may be null): the page numbers of the step's sequences by their place in the step, [n_seq, max_pages]:
  // row seq is row slots[seq] of page_table.  With it nothing here waits for the slot, and the number of a wave's first
  // page is asked for together with the position instead of after it (below).
  constexpr int HD = HEAD_DIM;
  constexpr int KS = (HD + 31) / 32;   // k steps of K Q^T (16x16x32)
  constexpr int DT = HD / 16;          // 16-row tiles of the output's head dimension
  constexpr int LS = HD + 2;           // floats a wave leaves in LDS per head: values, max, sum
  constexpr int KSLOTS = HD / 8;       // 16-byte pieces of a key row
  constexpr int KBYTES = PAGE * HD * 2, VBYTES = HD * PAGE * 2;   // a page's keys and values of one kv head
  constexpr int NLOAD = KBYTES / 1024;                            // 1 KB instructions for each of the two
  using KSw = SlotSwizzle<KSLOTS>;
  using VSw = SlotSwizzle<8>;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int split = blockIdx.z, seq = blockIdx.y;         // as attn_decode_kernel
  // The kv head of a block turns with its sequence and its share of the pages.  A block runs on the XCD that its linear
  // number mod 8 names; with the kv head straight from blockIdx.x and eight kv heads, an XCD would read one head for
  // good, and a head's keys and values lie at the same 8 KB (head size 64) of every 64 KB of the cache.  Whatever
  // address bits an L2 spreads its reads by, every XCD now sees all of them; the reads and sums are the same.
  const int kvh = (int)((blockIdx.x / head_blocks + seq + split) % (gridDim.x / head_blocks)), hb = blockIdx.x % head_blocks;
  // Which page a wave takes first depends on the sequence's length, which is a trip to memory away.  With the pages
  // listed by sequence their place is known at once, so every lane asks for a candidate now: lane s - 1 for the page the
  // wave would start at if the block's share were s pages (split * s + wave, without a window), and the one that the
  // position then calls for is picked from the lanes.  That makes position and page number one trip instead of two.
  const int first_wave = (int)(threadIdx.x >> 6);
  int candidate = -1;
  if (seq_pages != nullptr && window == 0) {
    const long long at = (long long)split * ((int)(threadIdx.x & 63) + 1) + first_wave;
    if (at < max_pages) candidate = seq_pages[(size_t)seq * max_pages + at];
  }
  const int pos = positions[seq];
  const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
  const int first_pg = lo / PAGE, last_pg = pos / PAGE;
  const int n_splits = sp.most, used = splits_used(sp, last_pg - first_pg + 1);
  const int span = (last_pg - first_pg + used) / used;
  const int pg0 = first_pg + split * span;
  const int pg1 = pg0 + span - 1 < last_pg ? pg0 + span - 1 : last_pg;
  if (pg0 > pg1) return;               // the whole block: fewer pages than splits
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = lane & 15, G = lane >> 4;
  const int hig = hb * 16 + j;                    // head within the group
  const int heads_here = group - hb * 16 < 16 ? group - hb * 16 : 16;
  const bool head_ok = j < heads_here;
  const int head = kvh * group + hig;
  const int32_t* my_pages = seq_pages != nullptr ? seq_pages + (size_t)seq * max_pages : page_table + (size_t)slots[seq] * max_pages;

  typedef __attribute__((address_space(3))) char lds_char;
  lds_char* wbuf = (lds_char*)lds + (size_t)wave * (KBYTES + VBYTES);      // this wave's page: keys, then values
  const uint32_t wbase = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)wbuf);
  // which piece of the page each lane fetches with load number c: the one that belongs at LDS slot c * 64 + lane
  uint32_t koff[NLOAD], voff[NLOAD];
#pragma unroll
  for (int c = 0; c < NLOAD; ++c) {
    const int L = c * 64 + lane;
    const int krow = L / KSLOTS, ks_ = L % KSLOTS;
    koff[c] = (uint32_t)(krow * (HD * 2) + ((ks_ ^ KSw::of(krow)) << 4));
    const int vrow = L >> 3, vs_ = L & 7;
    voff[c] = (uint32_t)(vrow * (PAGE * 2) + ((vs_ ^ VSw::of(vrow)) << 4));
  }
  auto issue = [&](int page) {
    const void* kp = uniform_ptr(cache + (size_t)page * page_stride + (size_t)kvh * PAGE * HD);
    const void* vp = uniform_ptr(cache + v_off + (size_t)page * page_stride + (size_t)kvh * HD * PAGE);
#pragma unroll
    for (int c = 0; c < NLOAD; ++c) page_to_lds(kp, koff[c], wbase + c * 1024);
#pragma unroll
    for (int c = 0; c < NLOAD; ++c) page_to_lds(vp, voff[c], wbase + KBYTES + c * 1024);
  };

  const float* cs = cos_t ? cos_t + (size_t)pos * (rot / 2) : nullptr;
  const float* sn = cos_t ? sin_t + (size_t)pos * (rot / 2) : nullptr;
  // the queries' loads stand in front of the first page's; what they are turned into is computed behind them
  Rot8In qin[KS];
  const bf16_t* qrow = q + (size_t)seq * ldq + (size_t)(head_ok ? head : kvh * group) * HD;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + G * 8 < HD ? ks * 32 + G * 8 : 0;
    qin[ks] = FUSED ? rot8_load(qrow, d0, cs, sn, rot, interleaved) : Rot8In{*(const uint4*)(qrow + d0)};
  }
  const int own = pos % PAGE;          // the token's own row in its page
  const int own_t = 2 * (own >> 5) + ((own >> 2) & 1), own_j = 4 * ((own >> 3) & 3) + (own & 3);     // where it sits in the score tiles
  // The wave that will take the sequence's last page also takes in the token's own key and value from the step's row:
  // it asks for them here, with the queries, so that they are in when the page is (asked for when the page is reached
  // they would be one more trip to memory in the middle of the kernel).
  const bool takes_own = FUSED && new_kv && pg1 == last_pg && (last_pg - pg0) % NWV == wave;
  Rot8In kin[KS];
  uint32_t v_own[DT];
  if (FUSED) {
    // (every lane of every wave makes these loads, a wave that does not take the token's own from the queries' row:
    // loads under a condition would each be waited for in turn)
    const bf16_t* row = q + (size_t)seq * ldq;
    const bf16_t* krow_new = takes_own ? row + k_col + (size_t)kvh * HD : qrow;
    const bf16_t* vrow_new = takes_own ? row + v_col + (size_t)kvh * HD : qrow;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + G * 8 < HD ? ks * 32 + G * 8 : 0;
      kin[ks] = rot8_load(krow_new, d0, cs, sn, rot, interleaved);
    }
#pragma unroll
    for (int d = 0; d < DT; ++d) v_own[d] = vrow_new[d * 16 + j];
  }
  int pg = pg0 + wave;
  int page_cur;
  if (seq_pages != nullptr && window == 0 && span <= WAVE)        // the candidate of lane span - 1 is page split * span + wave
    page_cur = pg <= pg1 ? __builtin_amdgcn_readlane(candidate, span - 1) : -1;
  else
    page_cur = pg <= pg1 ? __builtin_amdgcn_readfirstlane(my_pages[pg]) : -1;
  int page_next = pg + NWV <= pg1 ? my_pages[pg + NWV] : -1;
  if (page_cur >= 0) issue(page_cur);

  uint4 qf[KS], k_own[KS];
  bool have_q = false;
  f32x4_t o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  for (; pg <= pg1; pg += NWV) {
    const int page = page_cur;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the page is in LDS (and the next page's number is here)
    page_cur = __builtin_amdgcn_readfirstlane(page_next);
    if (page < 0) {                                      // a page that is not there holds no key
      page_next = pg + 2 * NWV <= pg1 ? my_pages[pg + 2 * NWV] : -1;
      if (page_cur >= 0) issue(page_cur);
      continue;
    }
    bf16_t* kpage = cache + (size_t)page * page_stride + (size_t)kvh * PAGE * HD;
    bf16_t* vpage = cache + v_off + (size_t)page * page_stride + (size_t)kvh * HD * PAGE;
    const int key0 = pg * PAGE;
    uint4 kf[4][KS];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int row = 32 * (t >> 1) + 8 * (j >> 2) + 4 * (t & 1) + (j & 3);       // the token that is row j of score tile t
      const lds_char* kr = wbuf + row * (HD * 2);
      const int sw = KSw::of(row);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        kf[t][ks] = (ks * 32 + G * 8 < HD) ? lds_read16(kr + (((ks * 4 + G) ^ sw) << 4)) : make_uint4(0, 0, 0, 0);
    }
    uint4 vf[2][DT];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const int row = d * 16 + j;
        vf[u][d] = lds_read16(wbuf + KBYTES + row * (PAGE * 2) + (((4 * u + G) ^ VSw::of(row)) << 4));
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the operands are in registers: the wave's part of LDS is free
    page_next = pg + 2 * NWV <= pg1 ? my_pages[pg + 2 * NWV] : -1;
    if (page_cur >= 0) issue(page_cur);
    if (!have_q) {
      have_q = true;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[ks] = !(head_ok && ks * 32 + G * 8 < HD) ? make_uint4(0, 0, 0, 0)
                 : rot8_apply(qin[ks], ks * 32 + G * 8, FUSED && cs != nullptr, rot, interleaved);
      if (takes_own && j == own_j) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          if (ks * 32 + G * 8 < HD) k_own[ks] = rot8_apply(kin[ks], ks * 32 + G * 8, cs != nullptr, rot, interleaved);
      }
    }
    if (FUSED && new_kv && pg == last_pg) {
      // the token's own key and value come from the step's row, not from the cache; head block 0 stores them
      if (j == own_j) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (t == own_t) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
              if (ks * 32 + G * 8 < HD) {
                kf[t][ks] = k_own[ks];
                if (hb == 0) *(uint4*)(kpage + (size_t)own * HD + ks * 32 + G * 8) = kf[t][ks];
              }
          }
      }
      if (G == ((own >> 3) & 3)) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
          if (u == (own >> 5)) {
#pragma unroll
            for (int d = 0; d < DT; ++d) {
              const bf16_t val = (bf16_t)v_own[d];
              uint32_t w4[4] = {vf[u][d].x, vf[u][d].y, vf[u][d].z, vf[u][d].w};
              const int e = own & 7;
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (i == (e >> 1)) w4[i] = (e & 1) ? ((w4[i] & 0x0000ffffu) | ((uint32_t)val << 16)) : ((w4[i] & 0xffff0000u) | val);
              vf[u][d] = make_uint4(w4[0], w4[1], w4[2], w4[3]);
              if (hb == 0) vpage[(size_t)(d * 16 + j) * PAGE + own] = val;
            }
          }
      }
    }
    f32x4_t s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      s[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[t][ks]), as_bf16x8(qf[ks]), s[t], 0, 0, 0);
    }
    // lane: head = lane%16; element v of tile t is key  key0 + 32 (t/2) + 8 G + 4 (t%2) + v
    const bool need_mask = key0 + PAGE - 1 > pos || key0 < lo;
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float sv = s[t][v] * scale_log2e;
        if (need_mask) {
          const int key = key0 + 32 * (t >> 1) + 8 * G + 4 * (t & 1) + v;
          sv = (key <= pos && key >= lo) ? sv : -INFINITY;
        }
        s[t][v] = sv;
        mx = fmaxf(mx, sv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(m, mx);      // finite: every page of the range holds a valid key
    const float alpha = fast_exp2(m - m_new);
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float p = fast_exp2(s[t][v] - m_new);
        s[t][v] = p;
        rs += p;
      }
    rs += __shfl_xor(rs, 16, WAVE);
    rs += __shfl_xor(rs, 32, WAVE);
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int d = 0; d < DT; ++d) o[d] *= alpha;
    const bool tail = key0 + PAGE - 1 > pos;   // keys beyond the sequence: their values must not reach the product
#pragma unroll
    for (int u = 0; u < 2; ++u) {              // 32 keys each: tiles 2u and 2u+1
      bf16x8_t pb;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pb[e] = (__bf16)s[2 * u][e];
        pb[4 + e] = (__bf16)s[2 * u + 1][e];
      }
      const int ka = key0 + 32 * u + 8 * G;    // the first of the lane's eight keys
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        uint4 a = vf[u][d];
        if (tail) {
          uint32_t* w4 = (uint32_t*)&a;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (ka + 2 * e > pos) w4[e] = 0;
            else if (ka + 2 * e + 1 > pos) w4[e] &= 0xffffu;
          }
        }
        o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), pb, o[d], 0, 0, 0);
      }
    }
  }
  __syncthreads();                      // every wave is done with its pages: the same LDS now takes the waves' results
  // each wave leaves (values, max, sum) per head in LDS; a wave that saw no page leaves (0, -inf, 0)
  if (head_ok) {
    float* dst = lds + (size_t)(wave * heads_here + j) * LS;
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[d * 16 + 4 * G + v] = o[d][v];
    if (G == 0) {
      dst[HD] = m;
      dst[HD + 1] = l;
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < heads_here * HD; idx += NWV * WAVE) {
    const int hh = idx / HD, d = idx - hh * HD;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NWV; ++w) M = fmaxf(M, lds[(size_t)(w * heads_here + hh) * LS + HD]);
    float L = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float* src = lds + (size_t)(w * heads_here + hh) * LS;
      const float wt = fast_exp2(src[HD] - M);
      L = fmaf(wt, src[HD + 1], L);
      acc = fmaf(wt, src[d], acc);
    }
    const int hd_ = kvh * group + hb * 16 + hh;
    if (n_splits == 1) {
      out[(size_t)seq * ldo + (size_t)hd_ * HD + d] = f32_to_bf16(acc / L);
    } else {
      float* dst = part + ((size_t)(seq * n_heads + hd_) * n_splits + split) * (HD + 4);
      dst[d] = acc;
      if (d == 0) {
        dst[HD] = M;
        dst[HD + 1] = L;
      }
    }
  }
}

// float32, one token per sequence, head sizes up to 128: attn_decode_kernel's arrangement (the pages of a split go to the
// block's waves in turn, all heads of the group are the MFMA's 16 columns, the waves merge through LDS in wave order)
// with v_mfma_f32_16x16x4_f32, a true float32 product, and expf.  A wave holds the keys and values of KT 16-key tiles
// at once (64 registers each, whatever the head size) and takes a page in 4 / KT such groups.
// Scores: MFMA row = key, column = head, and the four elements a lane holds of a 16-element chunk of the head are four
// k steps (the same elements on the key's and the query's side).  The scores land where the second product wants
// them: a lane's score of key 16 t + 4 G + v is the operand of k step (t, v), whose value operand is element v of the
// lane's 16 bytes of a transposed value row.
#include "exact_begin.h"      // the float32 kernel for steps of single tokens, and the merge of partial results
#if HEAD_DIM <= 128
template <int NWV>
__global__ __launch_bounds__(NWV* WAVE) void attn_decode_f32_kernel(
    const float* __restrict__ q, int ldq, float* __restrict__ out, int ldo, float* __restrict__ part,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, const int32_t* __restrict__ page_table,
    int max_pages, const float* __restrict__ cache, long long page_stride, long long v_off, int n_heads, int group,
    int head_blocks, SplitPlan sp, int window, float scale) {
  constexpr int HD = HEAD_DIM;
  constexpr int KC = HD / 16;          // 16-element chunks of the head
  constexpr int DT = HD / 16;          // 16-row tiles of the output's head dimension
  constexpr int KT = HD <= 64 ? 4 : 2; // 16-key tiles held at once
  constexpr int LS = HD + 2;           // floats a wave leaves in LDS per head: values, max, sum
  extern __shared__ float lds[];
  const int split = blockIdx.z, seq = blockIdx.y;         // as attn_decode_kernel
  const int kvh = blockIdx.x / head_blocks, hb = blockIdx.x % head_blocks;
  const int pos = positions[seq];
  const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
  const int first_pg = lo / PAGE, last_pg = pos / PAGE;
  const int n_splits = sp.most, used = splits_used(sp, last_pg - first_pg + 1);
  const int span = (last_pg - first_pg + used) / used;
  const int pg0 = first_pg + split * span;
  const int pg1 = pg0 + span - 1 < last_pg ? pg0 + span - 1 : last_pg;
  if (pg0 > pg1) return;               // the whole block: fewer pages than splits
  const int slot = slots[seq];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = lane & 15, G = lane >> 4;
  const int heads_here = group - hb * 16 < 16 ? group - hb * 16 : 16;
  const bool head_ok = j < heads_here;
  const int head = kvh * group + hb * 16 + j;

  float4 qf[KC];
  bool have_q = false;                 // the queries are read behind the first keys' loads
  f32x4_t o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  for (int pg = pg0 + wave; pg <= pg1; pg += NWV) {
    const int page = page_table[(size_t)slot * max_pages + pg];
    if (page < 0) continue;
    const float* kpage = cache + (size_t)page * page_stride + (size_t)kvh * PAGE * HD;
    const float* vpage = cache + v_off + (size_t)page * page_stride + (size_t)kvh * HD * PAGE;
#pragma unroll 1
    for (int kbase = 0; kbase < PAGE; kbase += KT * 16) {
      const int key0 = pg * PAGE + kbase;
      if (key0 > pos) break;                       // nothing but keys beyond the token from here on
      if (key0 + KT * 16 - 1 < lo) continue;       // nothing but keys before the window
      float4 kf[KT][KC];
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        const float* krow = kpage + (size_t)(kbase + t * 16 + j) * HD + 4 * G;
#pragma unroll
        for (int c = 0; c < KC; ++c) kf[t][c] = *(const float4*)(krow + 16 * c);
      }
      float4 vf[KT][DT];
#pragma unroll
      for (int t = 0; t < KT; ++t)
#pragma unroll
        for (int d = 0; d < DT; ++d) vf[t][d] = *(const float4*)(vpage + (size_t)(d * 16 + j) * PAGE + kbase + t * 16 + 4 * G);
      if (!have_q) {
        have_q = true;
        const float* qrow = q + (size_t)seq * ldq + (size_t)(head_ok ? head : kvh * group) * HD + 4 * G;
#pragma unroll
        for (int c = 0; c < KC; ++c) qf[c] = head_ok ? *(const float4*)(qrow + 16 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      f32x4_t s[KT];
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        s[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
          s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t][c].x, qf[c].x, s[t], 0, 0, 0);
          s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t][c].y, qf[c].y, s[t], 0, 0, 0);
          s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t][c].z, qf[c].z, s[t], 0, 0, 0);
          s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t][c].w, qf[c].w, s[t], 0, 0, 0);
        }
      }
      // lane: head = lane%16; element v of tile t is key  key0 + 16 t + 4 G + v.  At least one key of the group counts.
      const bool need_mask = key0 + KT * 16 - 1 > pos || key0 < lo;
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < KT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float sv = s[t][v] * scale;
          if (need_mask) {
            const int key = key0 + 16 * t + 4 * G + v;
            sv = (key <= pos && key >= lo) ? sv : -INFINITY;
          }
          s[t][v] = sv;
          mx = fmaxf(mx, sv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      const float m_new = fmaxf(m, mx);
      const float alpha = expf(m - m_new);
      float rs = 0.f;
#pragma unroll
      for (int t = 0; t < KT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float p = expf(s[t][v] - m_new);
          s[t][v] = p;
          rs += p;
        }
      rs += __shfl_xor(rs, 16, WAVE);
      rs += __shfl_xor(rs, 32, WAVE);
      l = l * alpha + rs;
      m = m_new;
#pragma unroll
      for (int d = 0; d < DT; ++d) o[d] *= alpha;
      const bool tail = key0 + KT * 16 - 1 > pos;    // keys beyond the sequence: their values must not reach the product
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        const int ka = key0 + 16 * t + 4 * G;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
          float4 a = vf[t][d];
          if (tail) {
            a.x = ka <= pos ? a.x : 0.f;
            a.y = ka + 1 <= pos ? a.y : 0.f;
            a.z = ka + 2 <= pos ? a.z : 0.f;
            a.w = ka + 3 <= pos ? a.w : 0.f;
          }
          o[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, s[t][0], o[d], 0, 0, 0);
          o[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, s[t][1], o[d], 0, 0, 0);
          o[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, s[t][2], o[d], 0, 0, 0);
          o[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, s[t][3], o[d], 0, 0, 0);
        }
      }
    }
  }
  // each wave leaves (values, max, sum) per head in LDS; a wave that saw no key leaves (0, -inf, 0)
  if (head_ok) {
    float* dst = lds + (size_t)(wave * heads_here + j) * LS;
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[d * 16 + 4 * G + v] = o[d][v];
    if (G == 0) {
      dst[HD] = m;
      dst[HD + 1] = l;
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < heads_here * HD; idx += NWV * WAVE) {
    const int hh = idx / HD, d = idx - hh * HD;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NWV; ++w) M = fmaxf(M, lds[(size_t)(w * heads_here + hh) * LS + HD]);
    float L = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float* src = lds + (size_t)(w * heads_here + hh) * LS;
      const float wt = expf(src[HD] - M);          // the block holds a key, so M is finite; a wave without one weighs 0
      L = fmaf(wt, src[HD + 1], L);
      acc = fmaf(wt, src[d], acc);
    }
    const int hd_ = kvh * group + hb * 16 + hh;
    if (n_splits == 1) {
      out[(size_t)seq * ldo + (size_t)hd_ * HD + d] = acc / L;
    } else {
      float* dst = part + ((size_t)(seq * n_heads + hd_) * n_splits + split) * (HD + 4);
      dst[d] = acc;
      if (d == 0) {
        dst[HD] = M;
        dst[HD + 1] = L;
      }
    }
  }
}
#endif

// grid (sequences, heads); merges the partials of the splits that hold keys of the token, in page order.  A lane takes
// one element of the head (and every lane the same maxima and sums).  Eight splits at a time, their loads issued before
// the token's position is known: which of them count is decided afterwards, so that the position and the partials
// cost one trip to memory, not three.
// NATURAL: the partials' maxima are natural exponents and expf is used (the float32 kernels'), else base-2 ones.
template <typename TO, bool NATURAL>
__global__ __launch_bounds__(WAVE) void attn_combine_kernel(const float* __restrict__ part, TO* __restrict__ out, int ldo,
                                                            const int32_t* __restrict__ positions, int n_heads,
                                                            SplitPlan sp, int window) {
  constexpr int HD = HEAD_DIM;
  constexpr int PS = HD + 4;
  constexpr int ND = (HD + WAVE - 1) / WAVE;           // elements of the head per lane
  const int seq = blockIdx.x, head = blockIdx.y, lane = threadIdx.x, n_splits = sp.most;
  const float* base = part + (size_t)(seq * n_heads + head) * n_splits * PS;
  const int pos = positions[seq];
  float M = -INFINITY, L = 0.f, acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.f;
  int s1 = 0;
  for (int c0 = 0; c0 < n_splits && c0 <= s1; c0 += 8) {
    float ms[8], ls[8], v[8][ND];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int sl = c0 + i < n_splits ? c0 + i : n_splits - 1;
      ms[i] = base[(size_t)sl * PS + HD];
      ls[i] = base[(size_t)sl * PS + HD + 1];
#pragma unroll
      for (int e = 0; e < ND; ++e) v[i][e] = base[(size_t)sl * PS + (e * WAVE + lane < HD ? e * WAVE + lane : HD - 1)];
    }
    if (c0 == 0) {
      const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
      const int n_pages = pos / PAGE - lo / PAGE + 1;
      const int used = splits_used(sp, n_pages);
      const int span = (n_pages - 1 + used) / used;
      s1 = (n_pages - 1) / span;                     // the last split that was given pages
    }
    float M_new = M;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (c0 + i <= s1) M_new = fmaxf(M_new, ms[i]);
    const float keep = merge_weight<NATURAL>(M - M_new);       // 0 at the first round (M = -inf, M_new finite: every split given pages holds a key)
    L *= keep;
#pragma unroll
    for (int e = 0; e < ND; ++e) acc[e] *= keep;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (c0 + i <= s1) {
        const float w = merge_weight<NATURAL>(ms[i] - M_new);
        L = fmaf(w, ls[i], L);
#pragma unroll
        for (int e = 0; e < ND; ++e) acc[e] = fmaf(w, v[i][e], acc[e]);
      }
    M = M_new;
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int e = 0; e < ND; ++e)
    if (e * WAVE + lane < HD) Elem<TO>::store(out + (size_t)seq * ldo + (size_t)head * HD + e * WAVE + lane, acc[e] * inv);
}

#include "exact_end.h"

extern "C" int dlgo_attention_head_dim() { return HEAD_DIM; }

// q: rows of the step [T, >= H*hd] (rotated); out [T, >= H*hd]; positions, tok_seq per token; slots per sequence.
extern "C" const char* dlgo_attention_rows(const void* q, int ldq, void* out, int ldo, int dtype, int n_tokens, int n_heads,
                                           int n_kv, int head_dim, const int32_t* positions, const int32_t* tok_seq,
                                           const int32_t* slots, const int32_t* page_table, int max_pages, const void* cache,
                                           long long page_stride, long long v_off, int window, float scale, int n_splits,
                                           float* part, long long part_elems, hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
  DLGO_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad head counts H=%d KV=%d", n_heads, n_kv);
  DLGO_REQUIRE(n_splits >= 1 && n_splits <= 65535, "attention: bad number of splits %d", n_splits);
  DLGO_REQUIRE(n_splits == 1 || (part && part_elems >= (long long)n_tokens * n_heads * n_splits * (HEAD_DIM + 4)),
               "attention: scratch for partial results too small");
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim, "attention: row strides too short");
  DLGO_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window or page table width");
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(((uintptr_t)cache & 15) == 0 && page_stride % epc == 0 && v_off % epc == 0, "attention: cache pages must be 16-byte aligned");
  if (n_tokens == 0) return nullptr;
  dim3 grid(n_tokens, n_heads, n_splits);
  const int group = n_heads / n_kv;
  if (dtype == DLGO_DTYPE_F32)
    hipLaunchKernelGGL(attn_rows_kernel<float>, grid, dim3(WAVE), 0, stream, (const float*)q, ldq, (float*)out, ldo, positions,
                       tok_seq, slots, page_table, max_pages, (const float*)cache, page_stride, v_off, group, window, scale,
                       n_splits, part);
  else if (dtype == DLGO_DTYPE_BF16)
    hipLaunchKernelGGL(attn_rows_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, positions,
                       tok_seq, slots, page_table, max_pages, (const bf16_t*)cache, page_stride, v_off, group, window, scale,
                       n_splits, part);
  else
    DLGO_FAIL("attention: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("attention_rows");
  if (n_splits > 1) {     // the rows are the "sequences" of the combine: one position each
    if (dtype == DLGO_DTYPE_F32)
      hipLaunchKernelGGL((attn_combine_kernel<float, true>), dim3(n_tokens, n_heads), dim3(WAVE), 0, stream, part, (float*)out, ldo,
                         positions, n_heads, SplitPlan{n_splits, n_splits, 0}, window);
    else
      hipLaunchKernelGGL((attn_combine_kernel<bf16_t, true>), dim3(n_tokens, n_heads), dim3(WAVE), 0, stream, part, (bf16_t*)out, ldo,
                         positions, n_heads, SplitPlan{n_splits, n_splits, 0}, window);
    DLGO_LAUNCH_CHECK("attention_combine");
  }
  return nullptr;
}

#define LOG2E 1.4426950408889634f

// bfloat16, every sequence's rows of this step: cu_q [n_seq+1], start_pos [n_seq] (length before the step), slots [n_seq].
extern "C" const char* dlgo_attention_prefill(const void* q, int ldq, void* out, int ldo, int n_seq, int max_q_len, int n_heads,
                                              int n_kv, int head_dim, const int32_t* cu_q, const int32_t* start_pos,
                                              const int32_t* slots, const int32_t* page_table, int max_pages, const void* cache,
                                              long long page_stride, long long v_off, int window, float scale,
                                              hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
  DLGO_REQUIRE(HEAD_DIM <= 256, "attention: the tiled kernel takes head sizes up to 256");
  DLGO_REQUIRE(n_seq >= 0 && max_q_len >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad sizes");
  const int group = n_heads / n_kv;
  DLGO_REQUIRE(group <= PF_ROWS, "attention: the tiled kernel takes up to %d query heads per kv head, got %d", PF_ROWS, group);
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim && ldq % 8 == 0 && ldo % 4 == 0, "attention: row strides");
  DLGO_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0 && ((uintptr_t)cache & 15) == 0 && page_stride % 8 == 0 && v_off % 8 == 0,
               "attention: operands must be 16-byte aligned");
  DLGO_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window or page table width");
  DLGO_REQUIRE(scale > 0.f, "attention: the tiled kernel takes a positive scale, got %g", (double)scale);
  if (n_seq == 0 || max_q_len == 0) return nullptr;
  const int bq = PF_ROWS / group;
  dim3 grid((max_q_len + bq - 1) / bq, n_seq, n_kv);
  hipLaunchKernelGGL(attn_prefill_kernel, grid, dim3(PF_THREADS * PF_TEAMS), 0, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, cu_q,
                     start_pos, slots, page_table, max_pages, (const bf16_t*)cache, page_stride, v_off, group, bq, window,
                     scale * LOG2E);
  DLGO_LAUNCH_CHECK("attention_prefill");
  return nullptr;
}

// float32, every sequence's rows of this step, head sizes up to 128: arguments as dlgo_attention_prefill.
extern "C" const char* dlgo_attention_prefill_f32(const void* q, int ldq, void* out, int ldo, int n_seq, int max_q_len, int n_heads,
                                                  int n_kv, int head_dim, const int32_t* cu_q, const int32_t* start_pos,
                                                  const int32_t* slots, const int32_t* page_table, int max_pages,
                                                  const void* cache, long long page_stride, long long v_off, int window,
                                                  float scale, hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
#if HEAD_DIM <= 128
  DLGO_REQUIRE(n_seq >= 0 && max_q_len >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad sizes");
  const int group = n_heads / n_kv;
  DLGO_REQUIRE(group <= PF32_THREADS, "attention: the float32 tiled kernel takes up to %d query heads per kv head, got %d", PF32_THREADS, group);
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim && ldq % 4 == 0 && ldo % 4 == 0, "attention: row strides");
  DLGO_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)cache & 15) == 0 && page_stride % 4 == 0 && v_off % 4 == 0,
               "attention: operands must be 16-byte aligned");
  DLGO_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window or page table width");
  if (n_seq == 0 || max_q_len == 0) return nullptr;
  const int bq = PF32_THREADS / group;
  dim3 grid((max_q_len + bq - 1) / bq, n_seq, n_kv);
  hipLaunchKernelGGL(attn_prefill_f32_kernel, grid, dim3(PF32_THREADS), 0, stream, (const float*)q, ldq, (float*)out, ldo, cu_q,
                     start_pos, slots, page_table, max_pages, (const float*)cache, page_stride, v_off, group, bq, window, scale);
  DLGO_LAUNCH_CHECK("attention_prefill_f32");
  return nullptr;
#else
  DLGO_FAIL("attention: the float32 tiled kernel takes head sizes up to 128, this library is built for %d", HEAD_DIM);
#endif
}

// bfloat16, one row per sequence.  With cos_t/sin_t ([table_rows, rot/2]) the rows q are unrotated and are rotated
// here; with new_kv they are [q | k | v] rows whose key (rotated) and value enter the product and the cache here.
// max_pages_used bounds the pages of any sequence of the step (a recorded
// launch passes the context's bound).  seq_pages (may be null): [n_seq, max_pages], row i = row slots[i] of page_table;
// the kernel that takes pages through LDS then reads the pages' numbers by sequence (see there).  part: float32 scratch, used when the pages are split over several
// blocks: n_seq * n_heads * n_splits * (hd + 4) with n_splits = dlgo_attention_decode_splits(...).
static void decode_plan(int n_pairs, int group, int max_pages_used, bool fused, bool through_lds, int* nwv, SplitPlan* plan) {
  const int heads_here = group < 16 ? group : 16;
  const int per_wave = heads_here * (HEAD_DIM + 2) * 4;      // bytes of LDS a wave needs for the merge
  // the registers a wave needs grow with the head size (a page's keys and values are held at once), and a block
  // of w waves leaves each 2048 / w of them; the variant that rotates needs about a third more
  int w = HEAD_DIM <= 64 ? 16 : (HEAD_DIM <= 128 ? 8 : 4);
  if (fused) w >>= 1;
  // pages through LDS: a wave's page (keys and values, 256 bytes per element of the head) times the waves within 128 KB
  if (through_lds) w = HEAD_DIM <= 32 ? 16 : (HEAD_DIM <= 64 ? 8 : (HEAD_DIM <= 128 ? 4 : 2));
  while (w > 1 && w * per_wave > 60 * 1024) w >>= 1;
  // enough blocks to fill the chip: with few (sequence, kv head) pairs each pair's pages go to several blocks
  int splits = n_pairs >= 256 ? 1 : (256 + n_pairs - 1) / n_pairs;
  if (splits > max_pages_used) splits = max_pages_used;
  const int to_fill = splits;
  // and enough that a block has at most sixteen pages a wave, so that one long sequence among short ones is not the
  // step's tail.  These are blocks for the longest sequence the launch allows, which for a recorded step is the longest
  // the cache allows: a shorter sequence uses fewer of them (splits_used)
  const int long_pages = w * 16;
  if (max_pages_used > long_pages && splits < (max_pages_used + long_pages - 1) / long_pages)
    splits = (max_pages_used + long_pages - 1) / long_pages;
  if (splits > 1 && w > 8 && !through_lds) w = 8;
  if (through_lds && splits > 1) {
    // more waves than a sequence can have pages: a wave without a page only adds to the merge.  Halve the waves of a
    // block (down to 4), then deal the pages to fewer blocks (one sequence at 2,000 to 4,000 tokens: 11.4 -> 10.0 us)
    while (w > 4 && splits * w > max_pages_used) w >>= 1;
    if (splits * w > max_pages_used) splits = (max_pages_used + w - 1) / w;
  }
  *nwv = w;
  plan->most = splits;
  plan->least = to_fill < splits ? to_fill : splits;
  plan->chunk = splits > to_fill ? w * 16 : 0;
}

// variant: 0 or 2 = the pages go through LDS, 1 = they are read straight into the operands' registers
extern "C" int dlgo_attention_decode_splits(int n_seq, int n_heads, int n_kv, int max_pages_used, int fused, int variant) {
  int nwv;
  SplitPlan plan;
  const int group = n_heads / n_kv;
  decode_plan(n_seq * n_kv * ((group + 15) / 16), group, max_pages_used, fused != 0, variant != 1, &nwv, &plan);
  return plan.most;
}

extern "C" const char* dlgo_attention_decode(const void* q, int ldq, void* out, int ldo, float* part, long long part_elems,
                                             int n_seq, int n_heads, int n_kv, int head_dim, const int32_t* positions,
                                             const int32_t* slots, const int32_t* page_table, int max_pages,
                                             int max_pages_used, void* cache, long long page_stride, long long v_off,
                                             int window, float scale, const float* cos_t, const float* sin_t, int table_rows,
                                             int rot, int interleaved, int new_kv, int variant, const int32_t* seq_pages,
                                             hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
  DLGO_REQUIRE(HEAD_DIM <= 256, "attention: the split kernel takes head sizes up to 256");
  DLGO_REQUIRE(variant >= 0 && variant <= 2, "attention: unknown variant %d of the split kernel", variant);
  DLGO_REQUIRE(n_seq >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad sizes");
  DLGO_REQUIRE(max_pages_used >= 1 && max_pages_used <= max_pages, "attention: bad bound on the pages of a sequence");
  DLGO_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attention: cos and sin tables come together");
  DLGO_REQUIRE(cos_t == nullptr || (rot % 16 == 0 && rot > 0 && rot <= head_dim && table_rows > 0),
               "attention: the fused rotation takes a rotated width that is a multiple of 16, got %d", rot);
  DLGO_REQUIRE(!new_kv || ldq >= (n_heads + 2 * n_kv) * head_dim, "attention: rows with new keys and values hold [q | k | v]");
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim && ldq % 8 == 0, "attention: row strides");
  DLGO_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)cache & 15) == 0 && page_stride % 8 == 0 && v_off % 8 == 0,
               "attention: operands must be 16-byte aligned");
  const int group = n_heads / n_kv;
  const int head_blocks = (group + 15) / 16;
  int nwv;
  SplitPlan plan;
  const bool fused = cos_t != nullptr || new_kv;
  const bool through_lds = variant != 1;
  decode_plan(n_seq * n_kv * head_blocks, group, max_pages_used, fused, through_lds, &nwv, &plan);
  const int n_splits = plan.most;
  DLGO_REQUIRE(n_splits == 1 || (part && part_elems >= (long long)n_seq * n_heads * n_splits * (HEAD_DIM + 4)),
               "attention: scratch for partial results too small");
  DLGO_REQUIRE((long long)n_kv * head_blocks <= 65535 && n_seq <= 65535 && n_heads <= 65535 && n_splits <= 65535, "attention: grid too large");
  if (n_seq == 0) return nullptr;
  const int heads_here = group < 16 ? group : 16;
  const size_t smem = (size_t)nwv * heads_here * (HEAD_DIM + 2) * 4;
  dim3 grid(n_kv * head_blocks, n_seq, n_splits);
#define DECODE_GO(W_, F_)                                                                                                      \
  hipLaunchKernelGGL((attn_decode_kernel<W_, F_>), grid, dim3(W_ * WAVE), smem, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo,  \
                     part, positions, slots, page_table, max_pages, (bf16_t*)cache, page_stride, v_off, n_heads, group,        \
                     head_blocks, plan, window, scale * LOG2E, cos_t, sin_t, rot, interleaved, new_kv,                    \
                     n_heads * head_dim, (n_heads + n_kv) * head_dim)
  if (through_lds) {
    const size_t pages = (size_t)nwv * 2 * PAGE * HEAD_DIM * 2;       // a page's keys and values of one kv head for every wave
    const size_t lds_bytes = pages > smem ? pages : smem;
#define DECODE_LDS_GO(W_, F_)                                                                                                  \
  do {                                                                                                                         \
    auto kernel = attn_decode_lds_kernel<W_, F_>;                                                                              \
    static bool raised = false;          /* more than 64 KB of LDS has to be asked for once per kernel */                      \
    if (!raised) {                                                                                                             \
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);         \
      if (e != hipSuccess) DLGO_FAIL("attention: cannot get %d bytes of LDS: %s", 160 * 1024, hipGetErrorString(e));           \
      raised = true;                                                                                                           \
    }                                                                                                                          \
    hipLaunchKernelGGL(kernel, grid, dim3(W_* WAVE), lds_bytes, stream, (const bf16_t*)q, ldq, (bf16_t*)out, ldo, part,        \
                       positions, slots, page_table, max_pages, (bf16_t*)cache, page_stride, v_off, n_heads, group,            \
                       head_blocks, plan, window, scale* LOG2E, cos_t, sin_t, rot, interleaved, new_kv,                    \
                       n_heads* head_dim, (n_heads + n_kv) * head_dim, seq_pages);                                             \
  } while (0)
    if (fused) {
      if (nwv == 16) DECODE_LDS_GO(16, true);
      else if (nwv == 8) DECODE_LDS_GO(8, true);
      else if (nwv == 4) DECODE_LDS_GO(4, true);
      else DECODE_LDS_GO(2, true);
    } else {
      if (nwv == 16) DECODE_LDS_GO(16, false);
      else if (nwv == 8) DECODE_LDS_GO(8, false);
      else if (nwv == 4) DECODE_LDS_GO(4, false);
      else DECODE_LDS_GO(2, false);
    }
#undef DECODE_LDS_GO
  } else if (fused) {
    if (nwv == 8) DECODE_GO(8, true);
    else if (nwv == 4) DECODE_GO(4, true);
    else if (nwv == 2) DECODE_GO(2, true);
    else DECODE_GO(1, true);
  } else {
    if (nwv == 16) DECODE_GO(16, false);
    else if (nwv == 8) DECODE_GO(8, false);
    else if (nwv == 4) DECODE_GO(4, false);
    else if (nwv == 2) DECODE_GO(2, false);
    else DECODE_GO(1, false);
  }
#undef DECODE_GO
  DLGO_LAUNCH_CHECK("attention_decode");
  if (n_splits > 1) {
    hipLaunchKernelGGL((attn_combine_kernel<bf16_t, false>), dim3(n_seq, n_heads), dim3(WAVE), 0, stream, part, (bf16_t*)out, ldo,
                       positions, n_heads, plan, window);
    DLGO_LAUNCH_CHECK("attention_combine");
  }
  return nullptr;
}

// float32, one row per sequence, head sizes up to 128: arguments as dlgo_attention_decode without the rotation; the
// scratch is sized by dlgo_attention_decode_splits(..., fused = 0).
extern "C" const char* dlgo_attention_decode_f32(const void* q, int ldq, void* out, int ldo, float* part, long long part_elems,
                                                 int n_seq, int n_heads, int n_kv, int head_dim, const int32_t* positions,
                                                 const int32_t* slots, const int32_t* page_table, int max_pages,
                                                 int max_pages_used, const void* cache, long long page_stride, long long v_off,
                                                 int window, float scale, hipStream_t stream) {
  DLGO_REQUIRE(head_dim == HEAD_DIM, "attention: this library is built for head size %d, got %d", HEAD_DIM, head_dim);
#if HEAD_DIM <= 128
  DLGO_REQUIRE(n_seq >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention: bad sizes");
  DLGO_REQUIRE(max_pages_used >= 1 && max_pages_used <= max_pages, "attention: bad bound on the pages of a sequence");
  DLGO_REQUIRE(ldq >= n_heads * head_dim && ldo >= n_heads * head_dim && ldq % 4 == 0, "attention: row strides");
  DLGO_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)cache & 15) == 0 && page_stride % 4 == 0 && v_off % 4 == 0,
               "attention: operands must be 16-byte aligned");
  DLGO_REQUIRE(window >= 0, "attention: bad window");
  const int group = n_heads / n_kv;
  const int head_blocks = (group + 15) / 16;
  int nwv;
  SplitPlan plan;
  decode_plan(n_seq * n_kv * head_blocks, group, max_pages_used, false, false, &nwv, &plan);
  const int n_splits = plan.most;
  if (nwv > 8) nwv = 8;                // a wave holds 128 registers of keys and values: two waves to a SIMD
  DLGO_REQUIRE(n_splits == 1 || (part && part_elems >= (long long)n_seq * n_heads * n_splits * (HEAD_DIM + 4)),
               "attention: scratch for partial results too small");
  DLGO_REQUIRE((long long)n_kv * head_blocks <= 65535 && n_seq <= 65535 && n_heads <= 65535 && n_splits <= 65535, "attention: grid too large");
  if (n_seq == 0) return nullptr;
  const int heads_here = group < 16 ? group : 16;
  const size_t smem = (size_t)nwv * heads_here * (HEAD_DIM + 2) * 4;
  dim3 grid(n_kv * head_blocks, n_seq, n_splits);
#define DECODE_GO(W_)                                                                                                         \
  hipLaunchKernelGGL((attn_decode_f32_kernel<W_>), grid, dim3(W_ * WAVE), smem, stream, (const float*)q, ldq, (float*)out, ldo, \
                     part, positions, slots, page_table, max_pages, (const float*)cache, page_stride, v_off, n_heads, group,  \
                     head_blocks, plan, window, scale)
  if (nwv == 8) DECODE_GO(8);
  else if (nwv == 4) DECODE_GO(4);
  else if (nwv == 2) DECODE_GO(2);
  else DECODE_GO(1);
#undef DECODE_GO
  DLGO_LAUNCH_CHECK("attention_decode_f32");
  if (n_splits > 1) {
    hipLaunchKernelGGL((attn_combine_kernel<float, true>), dim3(n_seq, n_heads), dim3(WAVE), 0, stream, part, (float*)out, ldo,
                       positions, n_heads, plan, window);
    DLGO_LAUNCH_CHECK("attention_combine");
  }
  return nullptr;
#else
  DLGO_FAIL("attention: the float32 split kernel takes head sizes up to 128, this library is built for %d", HEAD_DIM);
#endif
}

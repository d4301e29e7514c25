// Matrix products for a few rows of X (decode): Y[t, n] = sum_k X[t, k] * W[n, k] with up to 64 tokens t, where the
// time goes to streaming W once.  computerex/dlgo's mat-vec shader gives 4 rows of W to a workgroup and splits k over
// lanes (gpu/shaders/matvec_f32.comp:17-47); here:
//
//  * skinny_kernel: 16 (or 32, 64) rows of W per block, k split over the block's waves, 16x16 MFMA with W as the
//    row operand and the tokens as the column operand (bfloat16: v_mfma_f32_16x16x32_bf16; float32:
//    v_mfma_f32_16x16x4_f32, a true float32 product).  Optionally the RMSNorm of the float32 residual rows rides in
//    the product, so that the normed rows are never written.
//  * gemv_kernel: up to 8 tokens on the vector units; a wave streams whole rows of W.
//
// Every reduction order is a function of N and K alone: a row of Y never depends on the other rows of the step.
#include "gemm_common.h"
#include <initializer_list>

// ----------------------------------------------------------------------------
// weight-streaming kernel for up to 8 tokens
// ----------------------------------------------------------------------------
template <typename T> struct Chunk;
#if DLGO_ELEM == DLGO_DTYPE_BF16
template <> struct Chunk<bf16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void unpack(const uint4& u, float* f) {
    f[0] = __uint_as_float(u.x << 16);
    f[1] = __uint_as_float(u.x & 0xffff0000u);
    f[2] = __uint_as_float(u.y << 16);
    f[3] = __uint_as_float(u.y & 0xffff0000u);
    f[4] = __uint_as_float(u.z << 16);
    f[5] = __uint_as_float(u.z & 0xffff0000u);
    f[6] = __uint_as_float(u.w << 16);
    f[7] = __uint_as_float(u.w & 0xffff0000u);
  }
};
#endif
template <> struct Chunk<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void unpack(const uint4& u, float* f) {
    f[0] = __uint_as_float(u.x);
    f[1] = __uint_as_float(u.y);
    f[2] = __uint_as_float(u.z);
    f[3] = __uint_as_float(u.w);
  }
};

#define GEMV_WAVES 4
#define GEMV_ROWS 4   // rows of W per wave: two gate/up pairs

template <typename T, int TM, int EPI>
__global__ __launch_bounds__(GEMV_WAVES* WAVE) void gemv_kernel(const T* __restrict__ W, const T* __restrict__ X,
                                                                 void* __restrict__ Y, int N, int Tn, int K, int ldw, int ldx,
                                                                 int ldy) {
  constexpr int E = Chunk<T>::E;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * GEMV_WAVES + wave) * GEMV_ROWS;
  if (n0 >= N) return;
  const T* wrow[GEMV_ROWS];
#pragma unroll
  for (int r = 0; r < GEMV_ROWS; ++r) wrow[r] = W + (size_t)(n0 + r < N ? n0 + r : N - 1) * ldw;
  const T* xrow[TM];
#pragma unroll
  for (int m = 0; m < TM; ++m) xrow[m] = X + (size_t)(m < Tn ? m : Tn - 1) * ldx;

  float acc[GEMV_ROWS][TM];
#pragma unroll
  for (int r = 0; r < GEMV_ROWS; ++r)
#pragma unroll
    for (int m = 0; m < TM; ++m) acc[r][m] = 0.f;

  const int chunks = K / E;
  for (int c = lane; c < chunks; c += WAVE) {
    uint4 wv[GEMV_ROWS];
#pragma unroll
    for (int r = 0; r < GEMV_ROWS; ++r) wv[r] = *(const uint4*)(wrow[r] + (size_t)c * E);
    float xf[TM][E];
#pragma unroll
    for (int m = 0; m < TM; ++m) {
      const uint4 xv = *(const uint4*)(xrow[m] + (size_t)c * E);
      Chunk<T>::unpack(xv, xf[m]);
    }
#pragma unroll
    for (int r = 0; r < GEMV_ROWS; ++r) {
      float wf[E];
      Chunk<T>::unpack(wv[r], wf);
#pragma unroll
      for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[r][m] = fmaf(wf[e], xf[m][e], acc[r][m]);
    }
  }
#pragma unroll
  for (int r = 0; r < GEMV_ROWS; ++r)
#pragma unroll
    for (int m = 0; m < TM; ++m) acc[r][m] = wave_sum(acc[r][m]);
  // lane m writes token m
#pragma unroll
  for (int m = 0; m < TM; ++m)
    if (lane == m && m < Tn) epilogue4<T, EPI>(Y, ldy, N, m, n0, acc[0][m], acc[1][m], acc[2][m], acc[3][m]);
}

// ----------------------------------------------------------------------------
// MFMA kernel for a few rows of X (decode): 16 rows of W per block, k split over the waves
// ----------------------------------------------------------------------------
// A block owns 16 consecutive rows of W and every token of the step (up to 16 * TB).  Its NW waves take
// the 128-byte pieces of those rows in turn (wave w: pieces w, w + NW, ...), so together they stream the
// rows front to back; each piece is two 16x16 MFMA steps with W as the row operand and X as the column
// operand.  The waves' partial tiles are summed through LDS in wave order, then wave 0 runs the epilogue:
// a lane holds four consecutive n of one token, as in the tiled kernel.
//
// NORM: X is the float32 residual stream and the product is taken with rmsnorm(X) * norm_w without
// writing the normed rows: the column operand is X[t,k] * norm_w[k], the sum of squares of each token is
// gathered on the way, and 1/sqrt(mean + eps) multiplies the finished sums (it is a scalar per token).
template <typename T> struct Mma16;
#if DLGO_ELEM == DLGO_DTYPE_BF16
template <> struct Mma16<bf16_t> {
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x4_t& c) {
    union { uint4 u; bf16x8_t v; } ua, ub;
    ua.u = a;
    ub.u = b;
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua.v, ub.v, c, 0, 0, 0);
  }
  // 8 floats -> one 16-byte operand
  static __device__ __forceinline__ uint4 pack(const float* f) {
    union { uint4 u; bf16x8_t v; } x;
#pragma unroll
    for (int e = 0; e < 8; ++e) x.v[e] = (__bf16)f[e];
    return x.u;
  }
};
#endif
template <> struct Mma16<float> {
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x4_t& c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
  }
};

template <typename T, int NW, int R, int TB, int EPI, bool NORM>
__global__ __launch_bounds__(NW* WAVE) void skinny_kernel(const T* __restrict__ W, const void* __restrict__ Xv,
                                                           const float* __restrict__ norm_w, float eps, void* __restrict__ Y,
                                                           int N, int Tn, int K, int ldw, int ldx, int ldy) {
  constexpr int EPC = 16 / sizeof(T);          // elements of a 16-byte operand
  constexpr int PIECE = 8 * EPC;               // elements of a 128-byte piece of a row
  __shared__ float red[NW][16][17];
  __shared__ float ssq[NW][TB][16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, G = lane >> 4;
  const int n0 = blockIdx.x * 16 * R;          // R groups of 16 rows share every load of X
  const T* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) wrow[r] = W + (size_t)(n0 + r * 16 + j < N ? n0 + r * 16 + j : N - 1) * ldw;

  f32x4_t acc[R][TB];
  float ss[TB];
#pragma unroll
  for (int c = 0; c < TB; ++c) {
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    ss[c] = 0.f;
  }
  const int pieces = (K + PIECE - 1) / PIECE;
  // blocks start at different places of their rows, so that at any moment they ask different memory channels
  const int rot = (int)((blockIdx.x * 7u) % (unsigned)pieces);
#pragma unroll 4
  for (int pi = wave; pi < pieces; pi += NW) {
    const int p = pi + rot < pieces ? pi + rot : pi + rot - pieces;
#pragma unroll
    for (int h = 0; h < 2; ++h) {            // the two 64-byte halves of the piece
      const int k = p * PIECE + h * 4 * EPC + G * EPC;
      const bool in = k < K;
      uint4 a[R];
#pragma unroll
      for (int r = 0; r < R; ++r) a[r] = in ? *(const uint4*)(wrow[r] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int c = 0; c < TB; ++c) {
        const int t = c * 16 + j;
        uint4 b = make_uint4(0, 0, 0, 0);
        if (in && t < Tn) {
          if (NORM) {
            const float* xr = (const float*)Xv + (size_t)t * ldx + k;
            float f[EPC];
#pragma unroll
            for (int e = 0; e < EPC; e += 4) {
              const float4 x4 = *(const float4*)(xr + e);
              const float4 w4 = *(const float4*)(norm_w + k + e);
              ss[c] = fmaf(x4.x, x4.x, ss[c]);
              ss[c] = fmaf(x4.y, x4.y, ss[c]);
              ss[c] = fmaf(x4.z, x4.z, ss[c]);
              ss[c] = fmaf(x4.w, x4.w, ss[c]);
              f[e] = x4.x * w4.x;
              f[e + 1] = x4.y * w4.y;
              f[e + 2] = x4.z * w4.z;
              f[e + 3] = x4.w * w4.w;
            }
            b = Mma16<T>::pack(f);
          } else {
            b = *(const uint4*)((const T*)Xv + (size_t)t * ldx + k);
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) Mma16<T>::run(a[r], b, acc[r][c]);
      }
    }
  }
  // lane: token = 16 c + j, rows 16 r + 4 G + v.  Tile by tile the partial sums go to LDS and wave 0 adds them in
  // wave order and runs the epilogue.
  float scale[TB];
  if (NORM) {
#pragma unroll
    for (int c = 0; c < TB; ++c) {
      float s = ss[c];
      s += __shfl_xor(s, 16, WAVE);
      s += __shfl_xor(s, 32, WAVE);
      if (G == 0) ssq[wave][c][j] = s;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < TB; ++c) {
      float s = 0.f;
      for (int w = 0; w < NW; ++w) s += ssq[w][c][j];
      scale[c] = 1.0f / sqrtf(s / (float)K + eps);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int c = 0; c < TB; ++c) {
      if (NW > 1) {
        if (r + c) __syncthreads();          // wave 0 has read the tile before
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][4 * G + v][j] = acc[r][c][v];
        __syncthreads();
      }
      if (wave == 0) {
        float v[4];
        if (NW > 1) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = 0.f;
          for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] += red[w][4 * G + q][j];
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = acc[r][c][q];
        }
        if (NORM) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] *= scale[c];
        }
        const int t = c * 16 + j;
        if (t < Tn) epilogue4<T, EPI>(Y, ldy, N, t, n0 + r * 16 + 4 * G, v[0], v[1], v[2], v[3]);
      }
    }
}

// The same product for rows of W that are a whole number of kilobytes, with W going through LDS.  skinny_kernel reads
// W as 16 rows x 64 bytes per instruction, which is what the MFMA's row operand looks like; memory gives whole 1 KB runs
// about 20% faster on a matrix of tens of megabytes.  Here a block owns 16 rows, wave w their w-th kilobyte: sixteen
// global_load_lds_dwordx4, one row's kilobyte each, straight into the wave's own 16 KB of LDS, and the operands come back
// with ds_read_b128.  A row's 16-byte pieces sit at slot (piece ^ row), so that the sixteen rows a quarter wave reads at
// once lie in different banks; the lane that fills a slot fetches the piece that belongs there.  X, the sums over the
// waves and the epilogue are skinny_kernel's (up to 16 tokens).
static __device__ __forceinline__ void row_to_lds(const void* base, uint32_t voff, uint32_t lds_base) {
  // 16 bytes per lane from base + voff to LDS at lds_base + lane * 16 (lds_base travels in M0, the same for the wave)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(base) : "memory");
}
typedef uint32_t rows_u32x4_t __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ uint4 lds_operand(const __attribute__((address_space(3))) char* p) {
  const rows_u32x4_t v = *(const __attribute__((address_space(3))) rows_u32x4_t*)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}

// What a product may do for the norm that follows it, or take from the product before it (see
// dlgo_gemm_rows_leave_parts and dlgo_gemm_rows_scaled):
//   MODE 1 (with the epilogue that adds into the float32 residual rows): beside the new residual rows it leaves
//     x * norm_w of them in the run dtype, not yet scaled, and each group of 16 columns its share of every row's sum of
//     squares;
//   MODE 2: its X are such unscaled rows; the shares are added up in a fixed order and the scale 1/sqrt(sum/width + eps)
//     multiplies the finished sums (it is a scalar per token), before the epilogue.
constexpr int NORM_PARTS_MAX = 256;   // most shares of a row's sum of squares (a normed width of 4096)

struct NormParts {
  const float* norm_w;     // mode 1: the following norm's weights [N]
  void* unscaled;          // mode 1: [T, ld_unscaled] in the run dtype
  int ld_unscaled;
  float* parts;            // mode 1: written, mode 2: read; [T, n_parts]
  int n_parts;
  int width;               // mode 2: the normed width (the number of elements the shares were summed over)
  float eps;               // mode 2
};

// Mode 2's sums of squares: each token's shares are added up by 16 lanes, each its every 16th in order, then across
// the lanes in a fixed pattern.  ask() issues the loads (in front of W's, so that they are in when W's first are);
// leave() adds them up and leaves each token's sum in sumsq[16] (shared memory); a barrier has to follow.
template <int NW, int MODE>
struct NormShares {
  static constexpr int TOK_STEP = NW * WAVE / 16;     // tokens that the block takes at a time
  static constexpr int TOK_TURNS = (16 + TOK_STEP - 1) / TOK_STEP;
  static constexpr int SHARES = MODE == 2 ? NORM_PARTS_MAX / 16 : 1;
  float share[TOK_TURNS][SHARES];
  __device__ __forceinline__ void ask(const NormParts& np, int Tn) {
    if (MODE != 2) return;
    // every load is made, from a place that holds a share (the row's first) where none is wanted, and what is not
    // wanted is left out when the shares are added up: a load under a condition is waited for before the code after
    // it goes on, and W's loads, which stand behind these, would start a trip to memory late
#pragma unroll
    for (int turn = 0; turn < TOK_TURNS; ++turn) {
      const int t = turn * TOK_STEP + (threadIdx.x >> 4);
      const float* p = np.parts + (size_t)(t < Tn ? t : 0) * np.n_parts;
#pragma unroll
      for (int u = 0; u < SHARES; ++u) {
        const int i = u * 16 + (threadIdx.x & 15);
        share[turn][u] = p[i < np.n_parts ? i : 0];
      }
    }
  }
  __device__ __forceinline__ void leave(float* sumsq, const NormParts& np, int Tn) const {
    if (MODE != 2) return;
#pragma unroll
    for (int turn = 0; turn < TOK_TURNS; ++turn) {
      const int t = turn * TOK_STEP + (threadIdx.x >> 4);
      float sh = 0.f;
#pragma unroll
      for (int u = 0; u < SHARES; ++u) sh += (t < Tn && u * 16 + (int)(threadIdx.x & 15) < np.n_parts) ? share[turn][u] : 0.f;
      sh += __shfl_xor(sh, 1, WAVE);
      sh += __shfl_xor(sh, 2, WAVE);
      sh += __shfl_xor(sh, 4, WAVE);
      sh += __shfl_xor(sh, 8, WAVE);
      if ((threadIdx.x & 15) == 0 && t < 16) sumsq[t] = sh;
    }
  }
};

// Mode 1 reads, besides W and X, the residual values it adds to and the norm's weights.  They are asked for at the
// kernel's start (by wave 0, which runs the epilogue), so that they arrive while W streams in: asked for after the
// product they would cost the kernel one more trip to memory, a quarter of what a product of a few megabytes takes.
struct ResidualAhead {
  float y[4], w[4];
};
template <int MODE>
__device__ __forceinline__ ResidualAhead residual_ahead(const void* __restrict__ Y, int ldy, int N, int n_first, bool tok, int t_row,
                                                        const NormParts& np) {
  ResidualAhead a;
#pragma unroll
  for (int q = 0; q < 4; ++q) a.y[q] = a.w[q] = 0.f;
  if (MODE != 1 || (threadIdx.x >> 6) != 0 || !tok) return a;
  const int n = n_first + 4 * ((threadIdx.x & 63) >> 4);
  const float* y = (const float*)Y + (size_t)t_row * ldy + n;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    if (n + q < N) {
      a.y[q] = y[q];
      a.w[q] = np.norm_w[n + q];
    }
  return a;
}

// The end of a streamed product for one group of 16 rows: the waves' partial sums go through LDS (the rows' place, once
// every wave is done with them, which the caller's barrier has made sure of); wave 0 adds them in wave order and runs the
// epilogue.  lane: token t_row (the block's token lane % 16), rows 4 G + v of the group.  part_index: where this
// group's share goes (mode 1).
template <typename T, int NW, int EPI, int MODE>
__device__ __forceinline__ void stream_finish(float* red, const f32x4_t& acc, void* __restrict__ Y, int ldy, int N, int n_first,
                                              bool tok, float sc, const NormParts& np, int part_index, int t_row,
                                              const ResidualAhead& ahead, int rows_here = 16) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, G = lane >> 4;
#pragma unroll
  for (int v = 0; v < 4; ++v) red[(wave * 16 + 4 * G + v) * 17 + j] = acc[v];
  __syncthreads();
  if (wave != 0) return;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] += red[(w * 16 + 4 * G + q) * 17 + j];
  const int n = n_first + 4 * G;
  if (4 * G >= rows_here) tok = false;         // a block of 8 rows: the other half of the tile is nobody's
  if (MODE == 2) {
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] *= sc;
  }
  if (MODE == 1) {
    // EPI is the sum into the residual rows: the new values themselves, their product with the norm's weights, and
    // the share of these four columns in the row's sum of squares
    float p = 0.f;
    if (tok) {
      float* y = (float*)Y + (size_t)t_row * ldy + n;
      T* u = (T*)np.unscaled + (size_t)t_row * np.ld_unscaled + n;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (n + q < N) {
          const float x = ahead.y[q] + v[q];
          y[q] = x;
          p = fmaf(x, x, p);
          Elem<T>::store(u + q, x * ahead.w[q]);
        }
    }
    p += __shfl_xor(p, 16, WAVE);
    p += __shfl_xor(p, 32, WAVE);
    if (tok && G == 0) np.parts[(size_t)t_row * np.n_parts + part_index] = p;
  } else if (tok) {
    epilogue4<T, EPI>(Y, ldy, N, t_row, n, v[0], v[1], v[2], v[3]);
  }
}

template <typename T, int NW, int R, int EPI, int MODE>
__global__ __launch_bounds__(NW* WAVE) void skinny_stream_kernel(const T* __restrict__ W, const void* __restrict__ Xv,
                                                                  void* __restrict__ Y, int N, int Tn, int K, int ldw, int ldx,
                                                                  int ldy, NormParts np, int rows) {
  // rows: 16, or (R == 1 only) 8: a block takes half a tile's rows, so that a matrix of few rows still gives every
  // compute unit a block; the tile's other half is computed on whatever LDS holds and dropped
  constexpr int EPC = 16 / sizeof(T);          // elements of a 16-byte operand
  constexpr int CH = 1024 / sizeof(T);         // elements of a row's kilobyte
  constexpr int STEPS = 16;                    // MFMA steps of a kilobyte: four 16-byte pieces each
  typedef __attribute__((address_space(3))) char lds_char;
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  lds_char* wbuf = (lds_char*)lds_raw + (size_t)(threadIdx.x >> 6) * 16384;
  const uint32_t wbase = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)wbuf);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, G = lane >> 4;
  const int n0 = R == 1 ? blockIdx.x * rows : blockIdx.x * 16 * R;    // the block's R groups of 16 rows take the wave's operands of X in turn
  const bool tok = j < Tn;
  // the lane's operands of X, once for all the groups: token j, the wave's kilobyte of k
  uint4 b[STEPS];
  {
    const T* xr = (const T*)Xv + (size_t)(tok ? j : 0) * ldx + wave * CH + G * EPC;
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) b[s_] = *(const uint4*)(xr + s_ * 4 * EPC);
  }
  __shared__ float sumsq[16];
  NormShares<NW, MODE> shares;                 // mode 2: asked for here, in front of W's loads
  shares.ask(np, Tn);
  ResidualAhead ahead[R];                      // mode 1: likewise
#pragma unroll
  for (int r = 0; r < R; ++r) ahead[r] = residual_ahead<MODE>(Y, ldy, N, n0 + r * 16, tok, j, np);
  // load c brings row c's kilobyte of a group; the lane fetches the piece that belongs at its slot.  Rows beyond N repeat the last.
  const char* base = (const char*)uniform_ptr(W + (size_t)n0 * ldw + wave * CH);
  const uint32_t last_row = (uint32_t)(N - 1 - n0);
  auto issue = [&](int r) {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      if (R == 1 && c >= rows) break;
      const uint32_t row = (uint32_t)(16 * r + c) < last_row ? (uint32_t)(16 * r + c) : last_row;
      row_to_lds(base, row * (uint32_t)ldw * (uint32_t)sizeof(T) + (uint32_t)((lane ^ c) << 4), wbase + c * 1024);
    }
  };
  issue(0);
  f32x4_t acc[R];
  const lds_char* arow = wbuf + j * 1024;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // group r's kilobytes are in LDS (and X is here)
    if (r == 0 && !tok) {
#pragma unroll
      for (int s_ = 0; s_ < STEPS; ++s_) b[s_] = make_uint4(0, 0, 0, 0);
    }
    if (R == 1) {                                          // one group: multiply as the operands come from LDS
#pragma unroll
      for (int s_ = 0; s_ < STEPS; ++s_)
        Mma16<T>::run(lds_operand(arow + (((s_ * 4 + G) ^ j) << 4)), b[s_], acc[r]);
    } else {
      uint4 aop[STEPS];
#pragma unroll
      for (int s_ = 0; s_ < STEPS; ++s_) aop[s_] = lds_operand(arow + (((s_ * 4 + G) ^ j) << 4));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // ... and in registers: the next group's may take their place
      if (r + 1 < R) issue(r + 1);
#pragma unroll
      for (int s_ = 0; s_ < STEPS; ++s_) Mma16<T>::run(aop[s_], b[s_], acc[r]);
    }
  }
  shares.leave(sumsq, np, Tn);
  __syncthreads();
  const float sc = MODE == 2 ? 1.0f / sqrtf(sumsq[j] / (float)np.width + np.eps) : 1.f;
  float* red = (float*)lds_raw;                // [NW][16][17]
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r) __syncthreads();                    // wave 0 has read the group before
    stream_finish<T, NW, EPI, MODE>(red, acc[r], Y, ldy, N, n0 + r * 16, tok, sc, np, blockIdx.x * R + r, j, ahead[r], R == 1 ? rows : 16);
  }
}

// The same for rows of more kilobytes than a block has waves: wave w takes kilobytes w, w + NW, ... of the block's 16
// rows in turn (turns of them each), into the same 16 KB of LDS; the next one streams in while this one is multiplied,
// and its operands of X, which are asked for in front of it, wait in a second set of registers.
template <typename T, int NW, int EPI, int MODE>
__global__ __launch_bounds__(NW* WAVE) void skinny_stream_long_kernel(const T* __restrict__ W, const void* __restrict__ Xv,
                                                                       void* __restrict__ Y, int N, int Tn, int turns, int ldw,
                                                                       int ldx, int ldy, NormParts np) {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int CH = 1024 / sizeof(T);
  constexpr int STEPS = 16;
  typedef __attribute__((address_space(3))) char lds_char;
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  lds_char* wbuf = (lds_char*)lds_raw + (size_t)(threadIdx.x >> 6) * 16384;
  const uint32_t wbase = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)wbuf);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, G = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const bool tok = j < Tn;
  const T* xr = (const T*)Xv + (size_t)(tok ? j : 0) * ldx + G * EPC;
  const char* base = (const char*)uniform_ptr(W + (size_t)n0 * ldw);
  const uint32_t last_row = (uint32_t)(N - 1 - n0);
  uint32_t woff[16];                           // where load c of a kilobyte starts within it
#pragma unroll
  for (int c = 0; c < 16; ++c)
    woff[c] = ((uint32_t)c < last_row ? (uint32_t)c : last_row) * (uint32_t)ldw * (uint32_t)sizeof(T) + (uint32_t)((lane ^ c) << 4);
  auto ask = [&](int turn, uint4* b) {         // a turn's operands of X and its kilobytes of W
    const int k0 = (turn * NW + wave) * CH;
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) b[s_] = *(const uint4*)(xr + k0 + s_ * 4 * EPC);
    const uint32_t kb = (uint32_t)k0 * (uint32_t)sizeof(T);
#pragma unroll
    for (int c = 0; c < 16; ++c) row_to_lds(base, woff[c] + kb, wbase + c * 1024);
  };
  f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const lds_char* arow = wbuf + j * 1024;
  auto multiply = [&](int turn, const uint4* b, uint4* b_next) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // this turn's kilobytes are in LDS, its X in registers
    uint4 aop[STEPS];
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) aop[s_] = lds_operand(arow + (((s_ * 4 + G) ^ j) << 4));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // ... and in registers: the next turn's may take their place
    if (turn + 1 < turns) ask(turn + 1, b_next);
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) Mma16<T>::run(aop[s_], tok ? b[s_] : make_uint4(0, 0, 0, 0), acc);
  };
  __shared__ float sumsq[16];
  NormShares<NW, MODE> shares;
  shares.ask(np, Tn);
  const ResidualAhead ahead = residual_ahead<MODE>(Y, ldy, N, n0, tok, j, np);
  uint4 b0[STEPS], b1[STEPS];
  ask(0, b0);
  for (int turn = 0; turn < turns; turn += 2) {
    multiply(turn, b0, b1);
    if (turn + 1 < turns) multiply(turn + 1, b1, b0);
  }
  shares.leave(sumsq, np, Tn);
  __syncthreads();
  const float sc = MODE == 2 ? 1.0f / sqrtf(sumsq[j] / (float)np.width + np.eps) : 1.f;
  stream_finish<T, NW, EPI, MODE>((float*)lds_raw, acc, Y, ldy, N, n0, tok, sc, np, blockIdx.x, j, ahead);
}

// The same with the RMSNorm of the float32 residual rows riding in the product (see skinny_kernel).  A wave needs the
// part of every token's row that belongs to its kilobyte of k: it loads that part with all its lanes, 16 bytes each in
// whole runs (and the norm's weights once, not once per token), multiplies, gathers each token's sum of squares, and
// leaves the column operands in LDS behind its kilobytes of W, a kilobyte per token, pieces placed as W's are.  X's
// loads stand in front of W's in program order, so that working on X waits for X only while W streams in.
template <typename T, int NW, int R, int EPI>
__global__ __launch_bounds__(NW* WAVE) void skinny_stream_norm_kernel(const T* __restrict__ W, const float* __restrict__ X,
                                                                       const float* __restrict__ norm_w, float eps,
                                                                       void* __restrict__ Y, int N, int Tn, int K, int ldw,
                                                                       int ldx, int ldy) {
  constexpr int EPC = 16 / sizeof(T);          // elements of a 16-byte operand
  constexpr int CH = 1024 / sizeof(T);         // elements of a row's kilobyte
  constexpr int STEPS = 16;                    // MFMA steps of a kilobyte: four 16-byte pieces each
  constexpr int LPT = CH / 4 / WAVE;           // loads of four floats per lane that bring one token's part of x (2 or 1)
  typedef __attribute__((address_space(3))) char lds_char;
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  const int wstride = 16384 + Tn * 1024;       // a wave's LDS: its kilobytes of W, then a kilobyte of operands per token
  lds_char* wbuf = (lds_char*)lds_raw + (size_t)(threadIdx.x >> 6) * wstride;
  lds_char* xbuf = wbuf + 16384;
  const uint32_t wbase = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)wbuf);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 15, G = lane >> 4;
  const int n0 = blockIdx.x * 16 * R;          // the block's R groups of 16 rows take the wave's operands of X in turn
  const int k0 = wave * CH;                    // this wave's part of k
  // x first: load number c of a lane brings four floats of token c / LPT
  float4 xv[16 * LPT], wv[LPT];
#pragma unroll
  for (int u = 0; u < LPT; ++u) wv[u] = *(const float4*)(norm_w + k0 + (u * WAVE + lane) * 4);
#pragma unroll
  for (int c = 0; c < 16 * LPT; ++c) {
    const int t = c / LPT, u = c % LPT;
    xv[c] = t < Tn ? *(const float4*)(X + (size_t)t * ldx + k0 + (u * WAVE + lane) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const char* base = (const char*)uniform_ptr(W + (size_t)n0 * ldw + k0);
  const uint32_t last_row = (uint32_t)(N - 1 - n0);
  auto issue = [&](int r) {                    // group r's kilobytes: load c brings row 16 r + c (rows beyond N repeat the last)
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const uint32_t row = (uint32_t)(16 * r + c) < last_row ? (uint32_t)(16 * r + c) : last_row;
      row_to_lds(base, row * (uint32_t)ldw * (uint32_t)sizeof(T) + (uint32_t)((lane ^ c) << 4), wbase + c * 1024);
    }
  };
  issue(0);
  // x * w in the run dtype into LDS: four elements of token t at element (u * 64 + lane) * 4 of the wave's kilobyte, that
  // is piece p = that / EPC, which sits at slot p ^ t
  float ssum[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < LPT; ++u) {
      const float4 x4 = xv[t * LPT + u], w4 = wv[u];
      ss = fmaf(x4.x, x4.x, ss);
      ss = fmaf(x4.y, x4.y, ss);
      ss = fmaf(x4.z, x4.z, ss);
      ss = fmaf(x4.w, x4.w, ss);
      const int e0 = (u * WAVE + lane) * 4;
      const int piece = e0 / EPC, within = e0 % EPC;          // within: 0 or 4 (bfloat16), 0 (float32)
      lds_char* dst = xbuf + t * 1024 + ((piece ^ t) << 4) + within * (int)sizeof(T);
      if (t < Tn) {
        if constexpr (sizeof(T) == 4) {
          *(__attribute__((address_space(3))) rows_u32x4_t*)dst =
              rows_u32x4_t{__float_as_uint(x4.x * w4.x), __float_as_uint(x4.y * w4.y), __float_as_uint(x4.z * w4.z), __float_as_uint(x4.w * w4.w)};
        } else {
          const float f[4] = {x4.x * w4.x, x4.y * w4.y, x4.z * w4.z, x4.w * w4.w};
          typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
          *(__attribute__((address_space(3))) u32x2_t*)dst = u32x2_t{Elem<T>::pair(f[0], f[1]), Elem<T>::pair(f[2], f[3])};
        }
      }
    }
    ssum[t] = ss;
  }
  // the lane's column operands, once for all the groups of rows
  const bool tok = j < Tn;
  const lds_char* brow = xbuf + (tok ? j : 0) * 1024;
  uint4 bop[STEPS];
#pragma unroll
  for (int s_ = 0; s_ < STEPS; ++s_) {
    const rows_u32x4_t b4 = *(const __attribute__((address_space(3))) rows_u32x4_t*)(brow + (((s_ * 4 + G) ^ (tok ? j : 0)) << 4));
    bop[s_] = tok ? make_uint4(b4.x, b4.y, b4.z, b4.w) : make_uint4(0, 0, 0, 0);
  }
  f32x4_t acc[R];
  const lds_char* arow = wbuf + j * 1024;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // group r's kilobytes are in LDS
    uint4 aop[STEPS];
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) {
      const rows_u32x4_t a4 = *(const __attribute__((address_space(3))) rows_u32x4_t*)(arow + (((s_ * 4 + G) ^ j) << 4));
      aop[s_] = make_uint4(a4.x, a4.y, a4.z, a4.w);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // ... and in registers: the next group's may take their place
    if (r + 1 < R) issue(r + 1);
#pragma unroll
    for (int s_ = 0; s_ < STEPS; ++s_) Mma16<T>::run(aop[s_], bop[s_], acc[r]);
  }
  // each token's sum of squares over this wave's part of k, then everything through LDS as in the kernel above
#pragma unroll
  for (int t = 0; t < 16; ++t) ssum[t] = wave_sum(ssum[t]);
  __syncthreads();
  float* red = (float*)lds_raw;                // [NW][16][17]
  float* ssq = red + NW * 16 * 17;             // [NW][16]
#pragma unroll
  for (int t = 0; t < 16; ++t)
    if (lane == t) ssq[wave * 16 + t] = ssum[t];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r) __syncthreads();                    // wave 0 has read the group before
#pragma unroll
    for (int v = 0; v < 4; ++v) red[(wave * 16 + 4 * G + v) * 17 + j] = acc[r][v];
    __syncthreads();
    if (wave == 0) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] += red[(w * 16 + 4 * G + q) * 17 + j];
      float s2 = 0.f;
      for (int w = 0; w < NW; ++w) s2 += ssq[w * 16 + j];
      const float sc = 1.0f / sqrtf(s2 / (float)K + eps);
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] *= sc;
      if (tok) epilogue4<T, EPI>(Y, ldy, N, j, n0 + r * 16 + 4 * G, v[0], v[1], v[2], v[3]);
    }
  }
}

// Whether the streaming kernels take a product, and with how many waves: up to 16 tokens and rows of whole kilobytes.
// Rows of 2, 3, 4, 6 or 8 KB: a wave per kilobyte (a wave keeps 16 KB of LDS; eight of them fill a compute unit's),
// *turns = 1.  Other lengths, if some number of waves from 8 down to 4 divides them: each wave takes *turns kilobytes.
// Without `turns` (the kernel that stages the norm's rows in LDS) only the first kind.
template <typename T>
static int stream_waves(int Tn, int K, int ldw, int* turns = nullptr) {
  const long long bytes = (long long)K * sizeof(T);
  if (turns) *turns = 1;
  if (Tn < 1 || Tn > 16 || bytes % 1024 || bytes < 2048) return 0;
  if ((long long)ldw * sizeof(T) * 64 >= (1ll << 32)) return 0;      // row offsets within a block are 32 bits
  const int kb = (int)(bytes / 1024);
  if (kb == 2 || kb == 3 || kb == 4 || kb == 6 || kb == 8) return kb;
  if (!turns || kb > 8 * 64) return 0;
  for (int nw = 8; nw >= 4; --nw)
    if (kb % nw == 0) {
      *turns = kb / nw;
      return nw;
    }
  return 0;
}

// The compute units of the current device (asked once; 256 on the chip this is written for).
static int compute_units() {
  static int cus = 0;
  if (cus <= 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    else cus = 256;
  }
  return cus;
}

// Rows that a wave takes in several turns, or whose kilobytes are 5 or 7, go to the kernel with one group of rows a block.
static bool stream_is_long(int nw, int turns) { return turns > 1 || nw == 5 || nw == 7; }

// A block takes up to four groups of 16 rows in turn, which share its operands of X (and the work on the norm): as many
// as leave blocks for at least five eighths of the compute units (a function of N alone).  Measured with 1 to 16 tokens
// on matrices of 2,048 to 128,256 rows of 4 to 8 KB: fewer blocks than that cost more than the shared work saves; with
// more, four groups are 5 to 25% faster than one on the wide matrices and two on those of 5,000 to 6,000 rows.  (Where
// two blocks share a compute unit's LDS, rows of 4 KB, one group a block is 5% faster for the plain product of 16,384
// rows with up to 8 rows of X, 15.8 against 16.5 us; the product that applies a norm left to it adds up the norm's
// shares once per block and loses that again, 1.020 against 1.011 ms a step, so the rule has no such exception.)
// Rows of W a block of one group takes: 16, a whole MFMA tile, or 8 where tiles of 16 would give at most half of the
// compute units a block (an output projection of 2,048 rows: 128 blocks on 256 units; 4.3 to 4.9 against 4.5 to 5.3 us
// with 1 to 16 rows of X, a matrix of 1,024 rows 3.8 against 4.3 us) and, for the product that leaves a norm's shares,
// the shares of twice as many blocks still fit.  With more blocks than that, halves lose: 3,072 rows of 4 KB take 5.5
// to 7.3 us in blocks of 8 and 5.0 to 5.6 in blocks of 16, rows of 6 KB 8.2 against 6.2 us.
static int stream_rows(int N, bool is_long, int groups, int mode) {
  if (is_long || groups != 1 || (N + 15) / 16 > compute_units() / 2) return 16;
  if (mode == 1 && (N + 7) / 8 > NORM_PARTS_MAX) return 16;
  return 8;
}

static int stream_groups(int N, bool is_long) {
  const int blocks1 = (N + 15) / 16, fill = compute_units() * 5 / 8;
  return is_long ? 1 : (blocks1 >= 4 * fill ? 4 : (blocks1 >= 2 * fill ? 2 : 1));
}

template <typename T, int EPI, bool NORM, int MODE = 0>
static const char* launch_skinny_stream(const void* W, const void* X, const float* norm_w, float eps, void* Y, int N, int Tn, int K,
                                        int ldw, int ldx, int ldy, int nw, hipStream_t stream, NormParts np = NormParts{},
                                        int turns = 1, int force_groups = 0) {
  const bool is_long = stream_is_long(nw, turns);
  const int groups = force_groups && !is_long ? (force_groups > 0 ? force_groups : 1) : stream_groups(N, is_long);     // forced: tuning and tests
  const int rows = NORM || is_long ? 16 : (force_groups == -8 ? 8 : (force_groups == -16 ? 16 : stream_rows(N, is_long, groups, MODE)));
  dim3 g(groups == 1 ? (N + rows - 1) / rows : (N + 16 * groups - 1) / (16 * groups));
  // a wave's LDS: 16 KB of W and, with the norm, a kilobyte of column operands per token
  const int lds = nw * (16384 + (NORM ? Tn * 1024 : 0));
#define STREAM_RAISE(LIMIT_, ...)                                                                                               \
  do {                                                                                                                          \
    static bool raised = false;          /* 64 KB of LDS and more have to be asked for once per kernel */                       \
    if (!raised) {                                                                                                              \
      for (const void* k : {__VA_ARGS__}) {                                                                                     \
        hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, LIMIT_);                              \
        if (e != hipSuccess) DLGO_FAIL("gemm_rows: cannot get %d bytes of LDS: %s", LIMIT_, hipGetErrorString(e));              \
      }                                                                                                                         \
      raised = true;                                                                                                            \
    }                                                                                                                           \
  } while (0)
#define STREAM_LONG_GO(NW_)                                                                                                     \
  do {                                                                                                                          \
    if constexpr (!NORM) {                                                                                                      \
      auto kernel = skinny_stream_long_kernel<T, NW_, EPI, MODE>;                                                               \
      STREAM_RAISE(NW_ * 16384, (const void*)kernel);                                                                           \
      hipLaunchKernelGGL(kernel, g, dim3(NW_* WAVE), lds, stream, (const T*)W, X, Y, N, Tn, turns, ldw, ldx, ldy, np);          \
    } else {                                                                                                                    \
      DLGO_FAIL("gemm_rows: rows of %d KB are not streamed with a norm", nw * turns);                                           \
    }                                                                                                                           \
  } while (0)
#define STREAM_GO(NW_)                                                                                                          \
  do {                                                                                                                          \
    if constexpr (NORM) {                                                                                                       \
      auto k1 = skinny_stream_norm_kernel<T, NW_, 1, EPI>;                                                                      \
      auto k2 = skinny_stream_norm_kernel<T, NW_, 2, EPI>;                                                                      \
      auto k4 = skinny_stream_norm_kernel<T, NW_, 4, EPI>;                                                                      \
      STREAM_RAISE(160 * 1024, (const void*)k1, (const void*)k2, (const void*)k4);                                              \
      auto kernel = groups == 4 ? k4 : (groups == 2 ? k2 : k1);                                                                 \
      hipLaunchKernelGGL(kernel, g, dim3(NW_* WAVE), lds, stream, (const T*)W, (const float*)X, norm_w, eps, Y, N, Tn, K, ldw,  \
                         ldx, ldy);                                                                                             \
    } else {                                                                                                                    \
      auto k1 = skinny_stream_kernel<T, NW_, 1, EPI, MODE>;                                                                  \
      auto k2 = skinny_stream_kernel<T, NW_, 2, EPI, MODE>;                                                  \
      auto k4 = skinny_stream_kernel<T, NW_, 4, EPI, MODE>;                                                  \
      STREAM_RAISE(NW_ * 16384, (const void*)k1, (const void*)k2, (const void*)k4);                                             \
      auto kernel = groups == 4 ? k4 : (groups == 2 ? k2 : k1);                                                                 \
      hipLaunchKernelGGL(kernel, g, dim3(NW_* WAVE), lds, stream, (const T*)W, X, Y, N, Tn, K, ldw, ldx, ldy, np, rows);        \
    }                                                                                                                           \
  } while (0)
  if (is_long) {
    switch (nw) {
      case 2: STREAM_LONG_GO(2); break;
      case 3: STREAM_LONG_GO(3); break;
      case 4: STREAM_LONG_GO(4); break;
      case 5: STREAM_LONG_GO(5); break;
      case 6: STREAM_LONG_GO(6); break;
      case 7: STREAM_LONG_GO(7); break;
      default: STREAM_LONG_GO(8); break;
    }
    return nullptr;
  }
  switch (nw) {
    case 2: STREAM_GO(2); break;
    case 3: STREAM_GO(3); break;
    case 4: STREAM_GO(4); break;
    case 6: STREAM_GO(6); break;
    default: STREAM_GO(8); break;
  }
#undef STREAM_GO
#undef STREAM_LONG_GO
#undef STREAM_RAISE
  return nullptr;
}

template <typename T, int NW, int R, int EPI, bool NORM>
static void launch_skinny_nw(const void* W, const void* X, const float* norm_w, float eps, void* Y, int N, int Tn, int K, int ldw,
                             int ldx, int ldy, hipStream_t stream) {
  dim3 g((N + 16 * R - 1) / (16 * R)), b(NW * WAVE);
  const int tb = (Tn + 15) / 16;
#define SKINNY_GO(TB_) hipLaunchKernelGGL((skinny_kernel<T, NW, R, TB_, EPI, NORM>), g, b, 0, stream, (const T*)W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy)
  if (tb <= 1) SKINNY_GO(1);
  else if (tb == 2) SKINNY_GO(2);
  else if (tb == 3) SKINNY_GO(3);
  else SKINNY_GO(4);
#undef SKINNY_GO
}

// The number of waves that share a block's rows is a function of N and K alone, so the order of the sums does
// not depend on the step (few rows of long k: 16 waves, so that the few blocks keep more loads in flight).  force_nw (1, 2, 4, 8) is for tuning and tests.
template <typename T, int EPI, bool NORM>
static const char* launch_skinny(const void* W, const void* X, const float* norm_w, float eps, void* Y, int N, int Tn, int K, int ldw,
                                 int ldx, int ldy, hipStream_t stream, int force_nw = 0) {
  const int pieces = (K * (int)sizeof(T) + 127) / 128;
  int nw = pieces >= 128 && N <= 4096 ? 16 : (pieces >= 32 ? 8 : (pieces >= 16 ? 4 : (pieces >= 8 ? 2 : 1)));
  // rows of whole kilobytes and few tokens: W goes through LDS in whole 1 KB runs, where the matrix is large enough
  // for that to pay (force_nw 32 asks for it wherever it applies, 64 rules it out; other values choose the waves)
  int turns = 1;
  int sw = stream_waves<T>(Tn, K, ldw, NORM ? nullptr : &turns);
  if (NORM && sw * (16384 + Tn * 1024) > 160 * 1024) sw = 0;      // the tokens' operands have to fit in LDS beside W
  if (sw && (force_nw == 32 || force_nw == 0 || force_nw == 33 || force_nw == 34 || force_nw == 36 || force_nw == 40 || force_nw == 41)) {
    // 33, 34, 36: 1, 2, 4 groups of rows a block; 40, 41: one group, of 8 or 16 rows
    const int force = force_nw == 40 ? -8 : (force_nw == 41 ? -16 : (force_nw > 32 ? force_nw - 32 : 0));
    return launch_skinny_stream<T, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, sw, stream, NormParts{}, turns, force);
  }
  if (force_nw && force_nw < 32) nw = force_nw;
  // many rows: each block takes 2 or 4 groups of 16, which divides the traffic of X (a function of N alone)
  const bool wide = N >= 32768 && nw == 8, mid = N >= 8192 && nw == 8;
  if (nw == 16) launch_skinny_nw<T, 16, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (wide) launch_skinny_nw<T, 8, 4, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (mid) launch_skinny_nw<T, 8, 2, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 8) launch_skinny_nw<T, 8, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 4) launch_skinny_nw<T, 4, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 2) launch_skinny_nw<T, 2, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else launch_skinny_nw<T, 1, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  return nullptr;
}

template <typename T, int EPI>
static void launch_gemv(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                        hipStream_t stream) {
  const int blocks = (N + GEMV_WAVES * GEMV_ROWS - 1) / (GEMV_WAVES * GEMV_ROWS);
  dim3 g(blocks), b(GEMV_WAVES * WAVE);
  if (Tn == 1) hipLaunchKernelGGL((gemv_kernel<T, 1, EPI>), g, b, 0, stream, (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy);
  else if (Tn == 2) hipLaunchKernelGGL((gemv_kernel<T, 2, EPI>), g, b, 0, stream, (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy);
  else if (Tn <= 4) hipLaunchKernelGGL((gemv_kernel<T, 4, EPI>), g, b, 0, stream, (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy);
  else hipLaunchKernelGGL((gemv_kernel<T, 8, EPI>), g, b, 0, stream, (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy);
}

template <typename T, int EPI>
static const char* dispatch_rows(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int kind,
                                 hipStream_t stream) {
  // kind: 0 = the MFMA kernels, 1 = the vector kernel (at most 8 rows), 6..9 = the MFMA kernel that reads W into registers,
  // with 1, 2, 4, 8 waves per block, 10 = the MFMA kernel that sends W through LDS (where it applies, else as 0),
  // 11 = never that one, 15..17 = as 10 with 1, 2, 4 groups of weight rows a block, 18 and 19 = as 10 with one group of 8 or 16 rows
  if (kind == 1) {
    launch_gemv<T, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
    return nullptr;
  }
  return launch_skinny<T, EPI, false>(W, X, nullptr, 0.f, Y, N, Tn, K, ldw, ldx, ldy, stream,
                                      kind == 0 ? 0 : (kind == 10 ? 32 : (kind == 11 ? 64 : (kind >= 18 ? 22 + kind : (kind >= 15 ? 32 + (1 << (kind - 15)) : 1 << (kind - 6))))));
}

template <typename T>
static const char* rows_by_epilogue(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                                    int epi, int kind, hipStream_t stream) {
  switch (epi) {
    case EPI_STORE: return dispatch_rows<T, EPI_STORE>(W, X, Y, N, Tn, K, ldw, ldx, ldy, kind, stream);
    case EPI_ACCUM_F32: return dispatch_rows<T, EPI_ACCUM_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, kind, stream);
    case EPI_SWIGLU: return dispatch_rows<T, EPI_SWIGLU>(W, X, Y, N, Tn, K, ldw, ldx, ldy, kind, stream);
    case EPI_STORE_F32: return dispatch_rows<T, EPI_STORE_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, kind, stream);
    default: DLGO_FAIL("gemm_rows: unknown epilogue %d", epi);
  }
  return nullptr;
}

// Y[t, n] (epilogue) = sum_k X[t, k] W[n, k] for at most 64 rows of X.  ldy counts elements of Y's own type; for the
// SwiGLU epilogue Y has N/2 columns.
extern "C" const char* dlgo_gemm_rows(const void* W, const void* X, void* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                      int ldy, int epilogue, int kind, hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && Tn <= 64 && K > 0, "gemm_rows: bad sizes N=%d T=%d K=%d (at most 64 rows)", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm_rows: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(K % epc == 0, "gemm: inner size %d must be a multiple of %d for 16-byte loads", K, epc);
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ldw >= K && ldx >= K, "gemm: row strides (%d, %d) must be multiples of %d and at least K", ldw, ldx, epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0, "gemm: W and X must be 16-byte aligned");
  DLGO_REQUIRE(((uintptr_t)Y & 3) == 0 || (dtype == DLGO_DTYPE_BF16 && ((uintptr_t)Y & 1) == 0), "gemm: Y must be aligned to its elements");
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm: ldy %d shorter than N %d", ldy, N);
  DLGO_REQUIRE(kind == 0 || kind == 1 || (kind >= 6 && kind <= 11) || (kind >= 15 && kind <= 19), "gemm_rows: unknown kernel choice %d", kind);
  DLGO_REQUIRE(kind != 1 || Tn <= 8, "gemm: the vector kernel takes at most 8 rows, got %d", Tn);
  if (Tn == 0) return nullptr;
  const char* err = rows_by_epilogue<elem_t>(W, X, Y, N, Tn, K, ldw, ldx, ldy, epilogue, kind, stream);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_rows");
  return nullptr;
}

// Y (epilogue)= (rmsnorm(X) * norm_w) W^T for up to 64 rows of the float32 residual stream X [T, K], without
// writing the normed rows.  Epilogues as dlgo_gemm.
// kind: 0 = the kernel is chosen by the shape, 10 = W through LDS wherever that applies, 11 = never.
extern "C" const char* dlgo_gemm_rmsnorm(const void* W, const float* X, const float* norm_w, float eps, void* Y, int dtype, int N,
                                         int Tn, int K, int ldw, int ldx, int ldy, int epilogue, int kind, hipStream_t stream) {
  DLGO_REQUIRE(kind == 0 || kind == 10 || kind == 11, "gemm_rmsnorm: unknown kernel choice %d", kind);
  DLGO_REQUIRE(N > 0 && Tn >= 0 && Tn <= 64 && K > 0, "gemm_rmsnorm: bad sizes N=%d T=%d K=%d (at most 64 rows)", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm_rmsnorm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(K % epc == 0 && ldw % epc == 0 && ldx % 4 == 0 && ldw >= K && ldx >= K, "gemm_rmsnorm: K and the row strides must be multiples of %d", epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)norm_w & 15) == 0,
               "gemm_rmsnorm: W, X and the norm weight must be 16-byte aligned");
  DLGO_REQUIRE(eps > 0.f, "gemm_rmsnorm: eps must be positive");
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm_rmsnorm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm_rmsnorm: ldy %d shorter than N %d", ldy, N);
  if (Tn == 0) return nullptr;
  const int force = kind == 0 ? 0 : (kind == 10 ? 32 : 64);
#define NORM_GO(E_) launch_skinny<elem_t, E_, true>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream, force)
  const char* err = nullptr;
  switch (epilogue) {
    case EPI_STORE: err = NORM_GO(EPI_STORE); break;
    case EPI_ACCUM_F32: err = NORM_GO(EPI_ACCUM_F32); break;
    case EPI_SWIGLU: err = NORM_GO(EPI_SWIGLU); break;
    case EPI_STORE_F32: err = NORM_GO(EPI_STORE_F32); break;
    default: DLGO_FAIL("gemm_rmsnorm: unknown epilogue %d", epilogue);
  }
#undef NORM_GO
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_rmsnorm");
  return nullptr;
}


// Whether the streamed products take a product of Tn rows with a weight [N, K]: up to 16 rows of X, weight rows of whole
// kilobytes.  role 0: the plain product; 1: as dlgo_gemm_rows_leave_parts, which leaves a share of the sums of squares
// for every 16 of its N columns; 2: as dlgo_gemm_rows_scaled, which adds up the shares of the K columns it reads.  Both
// hold at most NORM_PARTS_MAX shares a row, so a normed width beyond 16 * NORM_PARTS_MAX is not theirs.
// How the streamed products would take a weight [N, K] with Tn rows of X: waves a block, the kilobytes of a row each wave
// takes in turn, and the groups of 16 weight rows a block works through (which share its reads of X).  Returns 0, with
// nothing written, if they do not take it.
extern "C" int dlgo_gemm_rows_stream_plan(int dtype, int N, int Tn, int K, int ldw, int* waves, int* turns, int* groups) {
  int t = 1;
  if (dtype != DLGO_ELEM || N <= 0) return 0;
  const int nw = stream_waves<elem_t>(Tn, K, ldw, &t);
  if (nw <= 0) return 0;
  *waves = nw;
  *turns = t;
  *groups = stream_groups(N, stream_is_long(nw, t));
  return 1;
}

extern "C" int dlgo_gemm_rows_streams(int dtype, int N, int Tn, int K, int ldw, int role) {
  int turns = 1;
  if (dtype != DLGO_ELEM || N <= 0 || stream_waves<elem_t>(Tn, K, ldw, &turns) <= 0) return 0;
  if (role == 1 && (N + 15) / 16 > NORM_PARTS_MAX) return 0;
  if (role == 2 && (K + 15) / 16 > NORM_PARTS_MAX) return 0;
  return role >= 0 && role <= 2 ? 1 : 0;
}

// residual [T, N] (float32) += X W^T, and for the norm that follows: unscaled [T, N] (run dtype) = new residual * norm_w,
// parts [T, n_parts] = every block's share of each row's sum of squares (n_parts = (N + 15) / 16, returned).  The consumer
// is dlgo_gemm_rows_scaled with these parts.
extern "C" const char* dlgo_gemm_rows_leave_parts(const void* W, const void* X, float* residual, int dtype, int N, int Tn, int K,
                                                  int ldw, int ldx, int ldy, const float* norm_w, void* unscaled, int ld_unscaled,
                                                  float* parts, long long parts_elems, int* n_parts, hipStream_t stream) {
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm_rows: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0 && ldw >= K && ldx >= K && ldy >= N && ld_unscaled >= N, "gemm_rows_leave_parts: bad sizes");
  int turns = 1;
  const int sw = stream_waves<elem_t>(Tn, K, ldw, &turns);
  DLGO_REQUIRE(sw > 0, "gemm_rows_leave_parts: up to 16 rows and weight rows of whole KB, got T=%d K=%d", Tn, K);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0,
               "gemm_rows_leave_parts: W and X must be 16-byte aligned with row strides that keep them so");
  DLGO_REQUIRE((N + 15) / 16 <= NORM_PARTS_MAX, "gemm_rows_leave_parts: a width of up to %d, got %d", 16 * NORM_PARTS_MAX, N);
  // a share for every block of one group of rows (16 rows, or 8: stream_rows), or for every group of a block of several
  const bool is_long = stream_is_long(sw, turns);
  const int groups = stream_groups(N, is_long);
  const int rows = stream_rows(N, is_long, groups, 1);
  const int np_ = groups == 1 ? (N + rows - 1) / rows : (N + 15) / 16;
  DLGO_REQUIRE(residual && norm_w && unscaled && parts && parts_elems >= (long long)Tn * np_, "gemm_rows_leave_parts: missing operand or scratch too small");
  *n_parts = np_;
  if (Tn == 0) return nullptr;
  NormParts np{norm_w, unscaled, ld_unscaled, parts, np_, 0, 0.f};
  const char* err = launch_skinny_stream<elem_t, EPI_ACCUM_F32, false, 1>(W, X, nullptr, 0.f, residual, N, Tn, K, ldw, ldx, ldy, sw, stream, np, turns);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_rows_leave_parts");
  return nullptr;
}

// Y (epilogue)= scale[t] * (X W^T) where X are rows that dlgo_gemm_rows_leave_parts left unscaled and
// scale[t] = 1 / sqrt(sum of the row's parts / width + eps).  Epilogues as dlgo_gemm_rows.
extern "C" const char* dlgo_gemm_rows_scaled(const void* W, const void* X, void* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                             int ldy, int epilogue, const float* parts, int n_parts, int width, float eps,
                                             hipStream_t stream) {
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm_rows: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0 && ldw >= K && ldx >= K, "gemm_rows_scaled: bad sizes");
  int turns = 1;
  const int sw = stream_waves<elem_t>(Tn, K, ldw, &turns);
  DLGO_REQUIRE(sw > 0, "gemm_rows_scaled: up to 16 rows and weight rows of whole KB, got T=%d K=%d", Tn, K);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0,
               "gemm_rows_scaled: W and X must be 16-byte aligned with row strides that keep them so");
  DLGO_REQUIRE(parts && n_parts > 0 && n_parts <= NORM_PARTS_MAX && width > 0 && eps > 0.f,
               "gemm_rows_scaled: parts, their number (up to %d, got %d), the width and eps", NORM_PARTS_MAX, n_parts);
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm: ldy %d shorter than N %d", ldy, N);
  if (Tn == 0) return nullptr;
  NormParts np{nullptr, nullptr, 0, const_cast<float*>(parts), n_parts, width, eps};
  const char* err = nullptr;
#define SCALED_GO(E_) err = launch_skinny_stream<elem_t, E_, false, 2>(W, X, nullptr, 0.f, Y, N, Tn, K, ldw, ldx, ldy, sw, stream, np, turns)
  switch (epilogue) {
    case EPI_STORE: SCALED_GO(EPI_STORE); break;
    case EPI_ACCUM_F32: SCALED_GO(EPI_ACCUM_F32); break;
    case EPI_SWIGLU: SCALED_GO(EPI_SWIGLU); break;
    case EPI_STORE_F32: SCALED_GO(EPI_STORE_F32); break;
    default: DLGO_FAIL("gemm_rows_scaled: unknown epilogue %d", epilogue);
  }
#undef SCALED_GO
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_rows_scaled");
  return nullptr;
}

#if DLGO_ELEM == DLGO_DTYPE_F32
#include "exact_end.h"
#endif

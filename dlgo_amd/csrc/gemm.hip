// Matrix products Y[t, n] = sum_k X[t, k] * W[n, k] for the projections of a
// step: W is a weight matrix [out, in] as the file stores it, X the rows of the
// step.  Both operands run along k in memory, which is what MFMA wants.
//
// computerex/dlgo has no GPU matrix-matrix product (gpu_batch_matvec falls back
// to one mat-vec, gpu/csrc/vulkan_gpu.c:1059-1069); its mat-vec shader gives 4
// rows to a workgroup and splits k over lanes (gpu/shaders/matvec_f32.comp:17-47),
// and its CPU path writes [nPos][rows] (blas/blas.go:422-494).  Two kernels here:
//
//  * gemm_kernel: LDS-tiled, one 32x32 MFMA tile grid per wave.  The MFMA "row"
//    side is W (i = n), the "column" side is X (j = t), so a lane ends up with
//    four consecutive n of one token: a vector store, and the two halves of a
//    gate/up pair when the rows of W interleave them.
//    bfloat16: v_mfma_f32_32x32x16_bf16.  float32: v_mfma_f32_32x32x2_f32, a
//    true float32 product with float32 accumulation.
//  * gemv_kernel: for a handful of tokens (decode).  A wave streams whole rows
//    of W with 16-byte loads; every lane keeps partial sums for each token.
//
// Epilogues: store in the run dtype; add into the float32 residual stream;
// SwiGLU of interleaved gate/up rows (out[t, f] = silu(y[2f]) * y[2f+1],
// ops/activation.go:8-19,36-38); store float32 (logits).
// Every reduction order is a function of k alone: a row of Y never depends on
// the other rows of the step.
#include "common.h"

enum { EPI_STORE = 0, EPI_ACCUM_F32 = 1, EPI_SWIGLU = 2, EPI_STORE_F32 = 3 };

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  // 16 bytes = 8 bfloat16 of k per lane: one 32x32x16 MFMA
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x16_t& c) {
    union { uint4 u; bf16x8_t v; } ua, ub;
    ua.u = a;
    ub.u = b;
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, c, 0, 0, 0);
  }
};
template <> struct Mma<float> {
  // 16 bytes = 4 float32 of k per lane: four 32x32x2 MFMAs
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x16_t& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};

// Four consecutive outputs n..n+3 of token t.
template <typename T, int EPI>
__device__ __forceinline__ void epilogue4(void* __restrict__ Y, int ldy, int N, int t, int n, float v0, float v1, float v2,
                                          float v3) {
  if (n >= N) return;
  const bool full = n + 3 < N;
  if (EPI == EPI_STORE) {
    T* y = (T*)Y + (size_t)t * ldy + n;
    if (full && (ldy & 3) == 0) {
      if (sizeof(T) == 4) {
        *(float4*)y = make_float4(v0, v1, v2, v3);
      } else {
        uint2 p;
        p.x = (uint32_t)f32_to_bf16(v0) | ((uint32_t)f32_to_bf16(v1) << 16);
        p.y = (uint32_t)f32_to_bf16(v2) | ((uint32_t)f32_to_bf16(v3) << 16);
        *(uint2*)y = p;
      }
    } else {
      const float v[4] = {v0, v1, v2, v3};
      for (int r = 0; r < 4 && n + r < N; ++r) Elem<T>::store(y + r, v[r]);
    }
  } else if (EPI == EPI_ACCUM_F32 || EPI == EPI_STORE_F32) {
    float* y = (float*)Y + (size_t)t * ldy + n;
    if (full && (ldy & 3) == 0) {
      float4 o = make_float4(v0, v1, v2, v3);
      if (EPI == EPI_ACCUM_F32) {
        const float4 old = *(float4*)y;
        o.x += old.x;
        o.y += old.y;
        o.z += old.z;
        o.w += old.w;
      }
      *(float4*)y = o;
    } else {
      const float v[4] = {v0, v1, v2, v3};
      for (int r = 0; r < 4 && n + r < N; ++r) y[r] = (EPI == EPI_ACCUM_F32 ? y[r] : 0.f) + v[r];
    }
  } else {   // EPI_SWIGLU: rows (n, n+1) and (n+2, n+3) are (gate, up) pairs; N is even
    T* y = (T*)Y + (size_t)t * ldy + (n >> 1);
    Elem<T>::store(y, silu_f(v0) * v1);
    if (n + 3 < N) Elem<T>::store(y + 1, silu_f(v2) * v3);
  }
}

// ----------------------------------------------------------------------------
// LDS-tiled MFMA kernel
// ----------------------------------------------------------------------------
#define GEMM_ROWB 144   // bytes of an LDS row: 128 of k and 16 of padding (spreads b128 reads over the banks)

template <typename T, int BN, int BT, int WN, int WT, int EPI>
__global__ __launch_bounds__(WN* WT* WAVE) void gemm_kernel(const T* __restrict__ W, const T* __restrict__ X,
                                                              void* __restrict__ Y, int N, int Tn, int K, int ldw, int ldx,
                                                              int ldy, int tiles_t) {
  constexpr int NT = WN * WT * WAVE;
  constexpr int EPC = 16 / sizeof(T);    // elements in a 16-byte chunk
  constexpr int BK = 128 / sizeof(T);    // k per tile
  constexpr int MI = BN / WN / 32, NJ = BT / WT / 32;
  constexpr int CA = BN * 8 / NT, CB = BT * 8 / NT;   // chunks per thread
  static_assert(BN * 8 % NT == 0 && BT * 8 % NT == 0, "tile does not divide over the threads");
  __shared__ __attribute__((aligned(16))) char lds[(BN + BT) * GEMM_ROWB];
  char* ldsA = lds;
  char* ldsB = lds + BN * GEMM_ROWB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wt = wave / WN;
  // consecutive blocks walk the tokens first: they share one tile of W
  const int tile_t = blockIdx.x % tiles_t, tile_n = blockIdx.x / tiles_t;
  const int n0 = tile_n * BN, t0 = tile_t * BT;

  f32x16_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[CA], rb[CB];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CA; ++i) {
      const int c = tid + i * NT, row = c >> 3, cc = c & 7;
      int n = n0 + row;
      n = n < N ? n : N - 1;
      const int k = k0 + cc * EPC;
      ra[i] = k < K ? *(const uint4*)(W + (size_t)n * ldw + k) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      const int c = tid + i * NT, row = c >> 3, cc = c & 7;
      int t = t0 + row;
      t = t < Tn ? t : Tn - 1;
      const int k = k0 + cc * EPC;
      rb[i] = k < K ? *(const uint4*)(X + (size_t)t * ldx + k) : make_uint4(0, 0, 0, 0);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < CA; ++i) {
      const int c = tid + i * NT;
      *(uint4*)(ldsA + (c >> 3) * GEMM_ROWB + (c & 7) * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      const int c = tid + i * NT;
      *(uint4*)(ldsB + (c >> 3) * GEMM_ROWB + (c & 7) * 16) = rb[i];
    }
  };

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    stash();
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);   // in flight while this tile is multiplied
    const char* pa = ldsA + (wn * (BN / WN) + (lane & 31)) * GEMM_ROWB + (lane >> 5) * 16;
    const char* pb = ldsB + (wt * (BT / WT) + (lane & 31)) * GEMM_ROWB + (lane >> 5) * 16;
#pragma unroll
    for (int slab = 0; slab < 4; ++slab) {
      uint4 a[MI], b[NJ];
#pragma unroll
      for (int i = 0; i < MI; ++i) a[i] = *(const uint4*)(pa + i * 32 * GEMM_ROWB + slab * 32);
#pragma unroll
      for (int j = 0; j < NJ; ++j) b[j] = *(const uint4*)(pb + j * 32 * GEMM_ROWB + slab * 32);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) Mma<T>::run(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

  // lane holds column j = lane%32 (token) and rows 8*(v/4) + 4*(lane/32) + v%4 (n) of each 32x32 tile
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int t = t0 + wt * (BT / WT) + j * 32 + (lane & 31);
    if (t >= Tn) continue;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * (BN / WN) + i * 32 + 8 * q + 4 * (lane >> 5);
        epilogue4<T, EPI>(Y, ldy, N, t, n, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
      }
    }
  }
}

// ----------------------------------------------------------------------------
// weight-streaming kernel for up to 8 tokens
// ----------------------------------------------------------------------------
template <typename T> struct Chunk;
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

// The number of waves that share a block's rows is a function of K alone, so the order of the sums does not
// depend on the step.  force_nw (1, 2, 4, 8) is for tuning and tests.
template <typename T, int EPI, bool NORM>
static void launch_skinny(const void* W, const void* X, const float* norm_w, float eps, void* Y, int N, int Tn, int K, int ldw,
                          int ldx, int ldy, hipStream_t stream, int force_nw = 0) {
  const int pieces = (K * (int)sizeof(T) + 127) / 128;
  int nw = pieces >= 32 ? 8 : (pieces >= 16 ? 4 : (pieces >= 8 ? 2 : 1));
  if (force_nw) nw = force_nw;
  // many rows: each block takes 2 or 4 groups of 16, which divides the traffic of X (a function of N alone)
  const bool wide = N >= 32768 && nw == 8, mid = N >= 8192 && nw == 8;
  if (wide) launch_skinny_nw<T, 8, 4, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (mid) launch_skinny_nw<T, 8, 2, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 8) launch_skinny_nw<T, 8, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 4) launch_skinny_nw<T, 4, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (nw == 2) launch_skinny_nw<T, 2, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else launch_skinny_nw<T, 1, 1, EPI, NORM>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream);
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
template <typename T, int BN, int BT, int WN, int WT, int EPI>
static void launch_tiled(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                         hipStream_t stream) {
  const int tiles_t = (Tn + BT - 1) / BT, tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL((gemm_kernel<T, BN, BT, WN, WT, EPI>), dim3((unsigned)(tiles_t * tiles_n)), dim3(WN * WT * WAVE), 0, stream,
                     (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy, tiles_t);
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
static void dispatch(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int force,
                     hipStream_t stream) {
  // force: 0 = choose, 1 = gemv, 2 = 128x128 tiles, 3 = 64x64, 4 = 32x32, 5 = 16 rows of W per block,
  // 6..9 = the same with 1, 2, 4, 8 waves per block
  int kind = force;
  if (kind == 0) {
    if (Tn <= 64) kind = 5;
    else {
      const long big = (long)((N + 127) / 128) * ((Tn + 127) / 128);
      const long mid = (long)((N + 63) / 64) * ((Tn + 63) / 64);
      kind = big >= 256 ? 2 : (mid >= 256 ? 3 : 4);
    }
  }
  if (kind == 1) launch_gemv<T, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (kind >= 5) launch_skinny<T, EPI, false>(W, X, nullptr, 0.f, Y, N, Tn, K, ldw, ldx, ldy, stream, kind == 5 ? 0 : 1 << (kind - 6));
  else if (kind == 2) launch_tiled<T, 128, 128, 2, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else if (kind == 3) launch_tiled<T, 64, 64, 2, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  else launch_tiled<T, 32, 32, 1, 1, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
}

template <typename T>
static const char* by_epilogue(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int epi,
                               int force, hipStream_t stream) {
  switch (epi) {
    case EPI_STORE: dispatch<T, EPI_STORE>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, stream); break;
    case EPI_ACCUM_F32: dispatch<T, EPI_ACCUM_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, stream); break;
    case EPI_SWIGLU: dispatch<T, EPI_SWIGLU>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, stream); break;
    case EPI_STORE_F32: dispatch<T, EPI_STORE_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, stream); break;
    default: DLGO_FAIL("gemm: unknown epilogue %d", epi);
  }
  return nullptr;
}

// Y[t, n] (epilogue) = sum_k X[t, k] W[n, k].  ldy counts elements of Y's own type; for the SwiGLU epilogue Y has N/2 columns.
extern "C" const char* dlgo_gemm(const void* W, const void* X, void* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                 int ldy, int epilogue, int force_kind, hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0, "gemm: bad sizes N=%d T=%d K=%d", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_DTYPE_F32 || dtype == DLGO_DTYPE_BF16, "gemm: unknown dtype code %d", dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(K % epc == 0, "gemm: inner size %d must be a multiple of %d for 16-byte loads", K, epc);
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ldw >= K && ldx >= K, "gemm: row strides (%d, %d) must be multiples of %d and at least K", ldw, ldx, epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)Y & 15) == 0, "gemm: operands must be 16-byte aligned");
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm: ldy %d shorter than N %d", ldy, N);
  DLGO_REQUIRE(force_kind >= 0 && force_kind <= 9, "gemm: unknown kernel choice %d", force_kind);
  DLGO_REQUIRE(force_kind != 1 || Tn <= 8, "gemm: the streaming kernel takes at most 8 rows, got %d", Tn);
  DLGO_REQUIRE(force_kind < 5 || Tn <= 64, "gemm: the 16-row kernel takes at most 64 rows of X, got %d", Tn);
  if (Tn == 0) return nullptr;
  const char* err = dtype == DLGO_DTYPE_F32 ? by_epilogue<float>(W, X, Y, N, Tn, K, ldw, ldx, ldy, epilogue, force_kind, stream)
                                            : by_epilogue<bf16_t>(W, X, Y, N, Tn, K, ldw, ldx, ldy, epilogue, force_kind, stream);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm");
  return nullptr;
}

// Y (epilogue)= (rmsnorm(X) * norm_w) W^T for up to 64 rows of the float32 residual stream X [T, K], without
// writing the normed rows.  Epilogues as dlgo_gemm.
extern "C" const char* dlgo_gemm_rmsnorm(const void* W, const float* X, const float* norm_w, float eps, void* Y, int dtype, int N,
                                         int Tn, int K, int ldw, int ldx, int ldy, int epilogue, hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && Tn <= 64 && K > 0, "gemm_rmsnorm: bad sizes N=%d T=%d K=%d (at most 64 rows)", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_DTYPE_F32 || dtype == DLGO_DTYPE_BF16, "gemm_rmsnorm: unknown dtype code %d", dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(K % epc == 0 && ldw % epc == 0 && ldx % 4 == 0 && ldw >= K && ldx >= K, "gemm_rmsnorm: K and the row strides must be multiples of %d", epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)Y & 15) == 0 && ((uintptr_t)norm_w & 15) == 0,
               "gemm_rmsnorm: operands must be 16-byte aligned");
  DLGO_REQUIRE(eps > 0.f, "gemm_rmsnorm: eps must be positive");
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm_rmsnorm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm_rmsnorm: ldy %d shorter than N %d", ldy, N);
  if (Tn == 0) return nullptr;
#define NORM_GO(T_, E_) launch_skinny<T_, E_, true>(W, X, norm_w, eps, Y, N, Tn, K, ldw, ldx, ldy, stream)
  if (dtype == DLGO_DTYPE_F32) {
    switch (epilogue) {
      case EPI_STORE: NORM_GO(float, EPI_STORE); break;
      case EPI_ACCUM_F32: NORM_GO(float, EPI_ACCUM_F32); break;
      case EPI_SWIGLU: NORM_GO(float, EPI_SWIGLU); break;
      case EPI_STORE_F32: NORM_GO(float, EPI_STORE_F32); break;
      default: DLGO_FAIL("gemm_rmsnorm: unknown epilogue %d", epilogue);
    }
  } else {
    switch (epilogue) {
      case EPI_STORE: NORM_GO(bf16_t, EPI_STORE); break;
      case EPI_ACCUM_F32: NORM_GO(bf16_t, EPI_ACCUM_F32); break;
      case EPI_SWIGLU: NORM_GO(bf16_t, EPI_SWIGLU); break;
      case EPI_STORE_F32: NORM_GO(bf16_t, EPI_STORE_F32); break;
      default: DLGO_FAIL("gemm_rmsnorm: unknown epilogue %d", epilogue);
    }
  }
#undef NORM_GO
  DLGO_LAUNCH_CHECK("gemm_rmsnorm");
  return nullptr;
}

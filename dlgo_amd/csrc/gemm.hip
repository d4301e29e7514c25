// Matrix products Y[t, n] = sum_k X[t, k] * W[n, k] for the projections of a step with many rows (prompts): W is a
// weight matrix [out, in] as the file stores it, X the rows of the step.  Both operands run along k in memory, which
// is what MFMA wants.  computerex/dlgo has no GPU matrix-matrix product (gpu_batch_matvec falls back to one mat-vec,
// gpu/csrc/vulkan_gpu.c:1059-1069); its CPU path writes [nPos][rows] (blas/blas.go:422-494).
//
// gemm_kernel: tiles of W and X go through LDS, two stages deep, so that a tile is fetched while the one before is
// multiplied; each wave owns a grid of 32x32 MFMA tiles.  The MFMA "row" side is W (i = n), the "column" side is X
// (j = t), so a lane ends up with four consecutive n of one token: a vector store, and the two halves of a gate/up
// pair when the rows of W interleave them.  bfloat16: v_mfma_f32_32x32x16_bf16.  float32: v_mfma_f32_32x32x2_f32, a
// true float32 product with float32 accumulation.  Blocks are numbered so that the blocks one XCD runs share tiles
// in that XCD's L2.
//
// gemm_direct_kernel: the same product for large shapes whose K is a whole number of 128-byte pieces.  Tiles go from
// memory straight into LDS (global_load_lds_dwordx4), without registers in between and two to three tiles ahead of
// the one being multiplied, so that neither the wait for memory nor the copy into LDS stands between the MFMAs.
//
// Every reduction order is a function of k alone: a row of Y never depends on the other rows of the step.
#include "gemm_common.h"

template <typename T> struct Mma;
#if DLGO_ELEM == DLGO_DTYPE_BF16
template <> struct Mma<bf16_t> {
  // 16 bytes = 8 bfloat16 of k per lane: one 32x32x16 MFMA
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x16_t& c) {
    union { uint4 u; bf16x8_t v; } ua, ub;
    ua.u = a;
    ub.u = b;
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.v, ub.v, c, 0, 0, 0);
  }
};
#endif
template <> struct Mma<float> {
  // 16 bytes = 4 float32 of k per lane: four 32x32x2 MFMAs
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, f32x16_t& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};


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
  constexpr int STAGE = (BN + BT) * GEMM_ROWB;
  static_assert(BN * 8 % NT == 0 && BT * 8 % NT == 0, "tile does not divide over the threads");
  extern __shared__ __attribute__((aligned(16))) char lds[];   // two stages of (BN + BT) rows

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wt = wave / WN;
  // Blocks go to the 8 XCDs in turn.  Renumber them so that each XCD gets a run of consecutive tiles, and let
  // consecutive tiles walk the tokens first: the blocks an XCD runs at a time share tiles of W in its L2.
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int tile_t = bid % tiles_t, tile_n = bid / tiles_t;
  const int n0 = tile_n * BN, t0 = tile_t * BT;

  f32x16_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  uint4 ra[CA], rb[CB];
  // Loads never branch: a chunk beyond K is read from the last chunk of the row and then replaced by zeros.
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CA; ++i) {
      const int c = tid + i * NT, row = c >> 3, cc = c & 7;
      int n = n0 + row;
      n = n < N ? n : N - 1;
      const int k = k0 + cc * EPC;
      const uint4 v = *(const uint4*)(W + (size_t)n * ldw + (k < K ? k : K - EPC));
      ra[i] = k < K ? v : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      const int c = tid + i * NT, row = c >> 3, cc = c & 7;
      int t = t0 + row;
      t = t < Tn ? t : Tn - 1;
      const int k = k0 + cc * EPC;
      const uint4 v = *(const uint4*)(X + (size_t)t * ldx + (k < K ? k : K - EPC));
      rb[i] = k < K ? v : make_uint4(0, 0, 0, 0);
    }
  };
  auto stash = [&](int stage) {
    char* ldsA = lds + stage * STAGE;
    char* ldsB = ldsA + BN * GEMM_ROWB;
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
  stash(0);
  __syncthreads();
  const int nk = (K + BK - 1) / BK;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) fetch((kt + 1) * BK);   // in flight while this tile is multiplied
    const char* pa = lds + cur * STAGE + (wn * (BN / WN) + (lane & 31)) * GEMM_ROWB + (lane >> 5) * 16;
    const char* pb = lds + cur * STAGE + BN * GEMM_ROWB + (wt * (BT / WT) + (lane & 31)) * GEMM_ROWB + (lane >> 5) * 16;
    // the operands of a slab are read from LDS while the slab before is multiplied
    uint4 a[2][MI], b[2][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i) a[0][i] = *(const uint4*)(pa + i * 32 * GEMM_ROWB);
#pragma unroll
    for (int j = 0; j < NJ; ++j) b[0][j] = *(const uint4*)(pb + j * 32 * GEMM_ROWB);
#pragma unroll
    for (int slab = 0; slab < 4; ++slab) {
      const int c = slab & 1, nx = c ^ 1;
      if (slab < 3) {
#pragma unroll
        for (int i = 0; i < MI; ++i) a[nx][i] = *(const uint4*)(pa + i * 32 * GEMM_ROWB + (slab + 1) * 32);
#pragma unroll
        for (int j = 0; j < NJ; ++j) b[nx][j] = *(const uint4*)(pb + j * 32 * GEMM_ROWB + (slab + 1) * 32);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) Mma<T>::run(a[c][i], b[c][j], acc[i][j]);
    }
    if (kt + 1 < nk) stash(cur ^ 1);          // the other stage was last read before the barrier below, one turn ago
    __syncthreads();
  }

  // A lane holds column j = lane%32 (token) and rows 8*(v/4) + 4*(lane/32) + v%4 (n) of each 32x32 tile: stores
  // from there would touch 64 rows of Y with a few bytes each.  Each tile is turned through a piece of LDS of the
  // wave's own (the stages are free after the last barrier), so that 8 lanes write 32 consecutive n of one token.
  float* turn = (float*)(lds + wave * (32 * GEMM_ROWB));
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *(float4*)(turn + (lane & 31) * (GEMM_ROWB / 4) + 8 * q + 4 * (lane >> 5)) =
            make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int tt = p * 8 + (lane >> 3), nn = (lane & 7) * 4;
        const float4 v = *(const float4*)(turn + tt * (GEMM_ROWB / 4) + nn);
        const int t = t0 + wt * (BT / WT) + j * 32 + tt;
        const int n = n0 + wn * (BN / WN) + i * 32 + nn;
        if (t < Tn) epilogue4<T, EPI>(Y, ldy, N, t, n, v.x, v.y, v.z, v.w);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

// 16 bytes per lane from base + voff into LDS at lds_base + lane * 16; lds_base is the same for the whole wave (it
// travels in M0).  Written as assembly so that the compiler does not make every later LDS read wait for these loads;
// wait_loads and the barrier below order them instead.
static __device__ __forceinline__ void load_to_lds(const void* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(base) : "memory");
}
template <int N> static __device__ __forceinline__ void wait_loads() {   // until at most N of this wave's loads are in flight
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// What a tiled product may do for the RMSNorm that follows it, or take from the product before it (the hand-off that
// gemm_rows.hip's streamed products have, for steps of many rows):
//   NORM 1 (with the epilogue that adds into the float32 residual rows): beside the new residual rows it leaves them times
//     the norm's weights in the run dtype, not yet scaled, and for every 32 columns their share of each row's sum of squares;
//   NORM 2: its X are such unscaled rows; every block adds up the shares of its rows in order and multiplies its sums by
//     1/sqrt(sum/width + eps) (a scalar per row, so it commutes with the product) before the epilogue.
struct TileNorm {
  const float* norm_w;     // NORM 1: the following norm's weights [N]
  void* unscaled;          // NORM 1: [T, ld_unscaled] in the run dtype
  int ld_unscaled;
  float* parts;            // NORM 1: written, NORM 2: read; [T, n_parts]
  int n_parts;
  int width;               // NORM 2: the normed width
  float eps;               // NORM 2
};

template <typename T, int BN, int BT, int WN, int WT, int NS, int EPI, int NORM = 0>
__global__ __launch_bounds__(WN* WT* WAVE) void gemm_direct_kernel(const T* __restrict__ W, const T* __restrict__ X,
                                                                     void* __restrict__ Yv, int N, int Tn, int K, int ldw, int ldx,
                                                                     int ldy, int tiles_t, int nk_split, long long split_stride,
                                                                     TileNorm tn) {
  constexpr int NW = WN * WT;
  constexpr int BK = 128 / sizeof(T);
  constexpr int MI = BN / WN / 32, NJ = BT / WT / 32;
  constexpr int LA = BN / 8 / NW, LB = BT / 8 / NW;     // loads (8 rows of 128 bytes each) per wave and stage
  constexpr int STAGE = (BN + BT) * 128;
  static_assert(BN % (8 * NW) == 0 && BT % (8 * NW) == 0, "tile does not divide over the waves");
  static_assert((NS - 2) * (LA + LB) < 64, "too many loads in flight for the counter");
  extern __shared__ __attribute__((aligned(16))) char lds[];   // NS stages of (BN + BT) rows of 128 bytes

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wt = wave / WN;
  int bid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);     // as in gemm_kernel
  const int tile_t = bid % tiles_t, tile_n = bid / tiles_t;
  const int n0 = tile_n * BN, t0 = tile_t * BT;

  f32x16_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // A load writes 1024 consecutive bytes of LDS: 8 rows without padding.  Row r therefore keeps its 16-byte piece p
  // at slot p ^ ((r >> 1) & 7), which spreads the 16 rows that a quarter of a wave reads at once over all banks; the
  // lane that fills slot s of row r fetches piece s ^ ((r >> 1) & 7).  Rows beyond the matrix repeat its last row.
  uint32_t offA[LA], offB[LB];
#pragma unroll
  for (int q = 0; q < LA; ++q) {
    const int r = (wave * LA + q) * 8 + (lane >> 3);
    const int p = (lane & 7) ^ ((r >> 1) & 7);
    int n = n0 + r;
    n = n < N ? n : N - 1;
    offA[q] = (uint32_t)(n - n0) * (uint32_t)ldw * (uint32_t)sizeof(T) + (uint32_t)p * 16u;
  }
#pragma unroll
  for (int q = 0; q < LB; ++q) {
    const int r = (wave * LB + q) * 8 + (lane >> 3);
    const int p = (lane & 7) ^ ((r >> 1) & 7);
    int t = t0 + r;
    t = t < Tn ? t : Tn - 1;
    offB[q] = (uint32_t)(t - t0) * (uint32_t)ldx * (uint32_t)sizeof(T) + (uint32_t)p * 16u;
  }
  // blockIdx.y: which run of nk_split k tiles this block sums (one run = the whole of k, unless the caller split it)
  const int kt0 = blockIdx.y * nk_split;
  const int nk = K / BK - kt0 < nk_split ? K / BK - kt0 : nk_split;
  void* Y = EPI == EPI_STORE_F32 ? (void*)((float*)Yv + (size_t)blockIdx.y * split_stride) : Yv;
  const char* baseA = (const char*)(W + (size_t)n0 * ldw) + (size_t)kt0 * 128;
  const char* baseB = (const char*)(X + (size_t)t0 * ldx) + (size_t)kt0 * 128;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const uint32_t ldsA = __builtin_amdgcn_readfirstlane(lds0 + wave * LA * 1024);
  const uint32_t ldsB = __builtin_amdgcn_readfirstlane(lds0 + BN * 128 + wave * LB * 1024);

  auto issue = [&](int kt, int stage) {
    const char* a = baseA + (size_t)kt * 128;
    const char* b = baseB + (size_t)kt * 128;
#pragma unroll
    for (int q = 0; q < LA; ++q) load_to_lds(a, offA[q], ldsA + stage * STAGE + q * 1024);
#pragma unroll
    for (int q = 0; q < LB; ++q) load_to_lds(b, offB[q], ldsB + stage * STAGE + q * 1024);
  };

#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < nk) issue(s, s);

  // NORM 2: the factor of each of the block's rows, while the first tiles are on their way (the loop's barriers stand
  // between this and the epilogue)
  __shared__ float row_scale[NORM == 2 ? BT : 1];
  if (NORM == 2) {
    for (int r = tid; r < BT; r += NW * WAVE) {
      const int t = t0 + r < Tn ? t0 + r : Tn - 1;
      const float* p = tn.parts + (size_t)t * tn.n_parts;
      float ss = 0.f;
      int q = 0;
      if ((tn.n_parts & 3) == 0 && ((uintptr_t)tn.parts & 15) == 0) {
        // 32 shares at a time, all their loads on the way before the first is added
        for (; q + 32 <= tn.n_parts; q += 32) {
          float4 v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = *(const float4*)(p + q + 4 * u);
#pragma unroll
          for (int u = 0; u < 8; ++u) ss += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        }
        for (; q + 4 <= tn.n_parts; q += 4) {
          const float4 v = *(const float4*)(p + q);
          ss += (v.x + v.y) + (v.z + v.w);
        }
      }
      for (; q < tn.n_parts; ++q) ss += p[q];
      row_scale[r] = 1.0f / sqrtf(ss / (float)tn.width + tn.eps);
    }
  }

  // operands: row lane%32 of a 32-row tile, pieces 2*slab + lane/32, found at slot (lane/32 ^ x) ^ 2*slab
  const int s0 = (lane >> 5) ^ ((lane >> 1) & 7);
  const int rowA = (wn * (BN / WN) + (lane & 31)) * 128, rowB = BN * 128 + (wt * (BT / WT) + (lane & 31)) * 128;
  int stage = 0;
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + NS - 2 < nk) wait_loads<(NS - 2) * (LA + LB)>();    // tile kt has arrived; the tiles after it may be on the way
    else wait_loads<0>();
    __syncthreads();        // ... for every wave, and every wave is done with tile kt-1, whose stage is filled next
    if (kt + NS - 1 < nk) {
      int ws = stage + NS - 1;
      ws = ws >= NS ? ws - NS : ws;
      issue(kt + NS - 1, ws);
    }
    const char* pa = lds + stage * STAGE + rowA;
    const char* pb = lds + stage * STAGE + rowB;
    uint4 a[2][MI], b[2][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i) a[0][i] = *(const uint4*)(pa + i * 32 * 128 + s0 * 16);
#pragma unroll
    for (int j = 0; j < NJ; ++j) b[0][j] = *(const uint4*)(pb + j * 32 * 128 + s0 * 16);
#pragma unroll
    for (int slab = 0; slab < 4; ++slab) {
      const int c = slab & 1, nx = c ^ 1;
      if (slab < 3) {
        const int so = (s0 ^ (2 * (slab + 1))) * 16;
#pragma unroll
        for (int i = 0; i < MI; ++i) a[nx][i] = *(const uint4*)(pa + i * 32 * 128 + so);
#pragma unroll
        for (int j = 0; j < NJ; ++j) b[nx][j] = *(const uint4*)(pb + j * 32 * 128 + so);
      }
      // the reads of the next slab stay in front of this slab's products: they arrive while these run
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) Mma<T>::run(a[c][i], b[c][j], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    stage = stage + 1 == NS ? 0 : stage + 1;
  }
  __syncthreads();      // the stages are free

  // bfloat16 results leave as whole rows: every wave puts its converted tiles into one [BT][OC] tile in the stages,
  // then the block stores it in pieces of 16 bytes, a row of the tile after the other (256 bytes in one run instead of
  // the 32 or 64 that a wave's own tile has per token).
  constexpr int OC = EPI == EPI_SWIGLU ? BN / 2 : BN;      // columns of Y that the block's tile has
  constexpr int OROW = OC * 2 + 16;                        // bytes of a row of it in LDS
  if constexpr (sizeof(T) == 2 && (EPI == EPI_STORE || EPI == EPI_SWIGLU) && BT * OROW <= NS * STAGE) {
    const int n_out = EPI == EPI_SWIGLU ? N >> 1 : N, c0 = EPI == EPI_SWIGLU ? n0 >> 1 : n0;
    if ((ldy & 7) == 0 && (n_out & 7) == 0 && ((uintptr_t)Y & 15) == 0) {
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int tl = wt * (BT / WT) + j * 32 + (lane & 31);
            const int nl = wn * (BN / WN) + i * 32 + 8 * q + 4 * (lane >> 5);     // four consecutive n of that token
            float v0 = acc[i][j][4 * q], v1 = acc[i][j][4 * q + 1], v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
            if (NORM == 2) {
              const float sc = row_scale[tl];
              v0 *= sc;
              v1 *= sc;
              v2 *= sc;
              v3 *= sc;
            }
            if (EPI == EPI_SWIGLU) {
              Elem<T>::store2((T*)(lds + tl * OROW + nl), silu_f<T>(v0) * v1, silu_f<T>(v2) * v3);
            } else {
              Elem<T>::store4((T*)(lds + tl * OROW + nl * 2), v0, v1, v2, v3);
            }
          }
      __syncthreads();
      constexpr int CPR = OC / 8;     // pieces of 16 bytes in a row
      for (int c = tid; c < BT * CPR; c += NW * WAVE) {
        const int row = c / CPR, piece = c % CPR;
        const int t = t0 + row, col = c0 + piece * 8;
        if (t < Tn && col < n_out) *(uint4*)((T*)Y + (size_t)t * ldy + col) = *(const uint4*)(lds + row * OROW + piece * 16);
      }
      return;
    }
  }

  // otherwise each wave turns its tiles through a piece of the stages, as in gemm_kernel
  float* turn = (float*)(lds + wave * (32 * GEMM_ROWB));
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *(float4*)(turn + (lane & 31) * (GEMM_ROWB / 4) + 8 * q + 4 * (lane >> 5)) =
            make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int tt = p * 8 + (lane >> 3), nn = (lane & 7) * 4;
        float4 v = *(const float4*)(turn + tt * (GEMM_ROWB / 4) + nn);
        const int t = t0 + wt * (BT / WT) + j * 32 + tt;
        const int n = n0 + wn * (BN / WN) + i * 32 + nn;
        if (NORM == 2) {
          const float sc = row_scale[wt * (BT / WT) + j * 32 + tt];
          v.x *= sc;
          v.y *= sc;
          v.z *= sc;
          v.w *= sc;
        }
        if (NORM == 1) {
          // the eight lanes of a token hold the 32 columns of this tile: the new residual values, their products with
          // the norm's weights, and the columns' share of the row's sum of squares (N is a multiple of 32 here)
          float ssq = 0.f;
          if (t < Tn && n < N) {
            float* y = (float*)Y + (size_t)t * ldy + n;
            const float4 old = *(const float4*)y;
            const float4 r = make_float4(old.x + v.x, old.y + v.y, old.z + v.z, old.w + v.w);
            *(float4*)y = r;
            const float4 w4 = *(const float4*)(tn.norm_w + n);
            Elem<T>::store4((T*)tn.unscaled + (size_t)t * tn.ld_unscaled + n, r.x * w4.x, r.y * w4.y, r.z * w4.z, r.w * w4.w);
            ssq = fmaf(r.x, r.x, fmaf(r.y, r.y, fmaf(r.z, r.z, r.w * r.w)));
          }
          ssq += __shfl_xor(ssq, 1, WAVE);
          ssq += __shfl_xor(ssq, 2, WAVE);
          ssq += __shfl_xor(ssq, 4, WAVE);
          if ((lane & 7) == 0 && t < Tn && n < N) tn.parts[(size_t)t * tn.n_parts + (n >> 5)] = ssq;
        } else if (t < Tn) {
          epilogue4<T, EPI>(Y, ldy, N, t, n, v.x, v.y, v.z, v.w);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <typename T, int BN, int BT, int WN, int WT, int NS, int EPI, int NORM = 0>
static const char* launch_direct(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                                 hipStream_t stream, int splits = 1, long long split_stride = 0, TileNorm tn = TileNorm{}) {
  const int tiles_t = (Tn + BT - 1) / BT, tiles_n = (N + BN - 1) / BN;
  const int nk_all = K / (int)(128 / sizeof(T)), nk_split = (nk_all + splits - 1) / splits;
  constexpr int smem = NS * (BN + BT) * 128;
  static_assert(smem >= WN * WT * 32 * GEMM_ROWB, "the stages must hold the waves' turning space");
  auto kernel = gemm_direct_kernel<T, BN, BT, WN, WT, NS, EPI, NORM>;
  static bool raised = false;
  if (smem > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) DLGO_FAIL("gemm: cannot get %d bytes of LDS: %s", smem, hipGetErrorString(e));
    raised = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_t * tiles_n), (unsigned)((nk_all + nk_split - 1) / nk_split)), dim3(WN * WT * WAVE),
                     smem, stream, (const T*)W, (const T*)X, Y, N, Tn, K, ldw, ldx, ldy, tiles_t, nk_split, split_stride, tn);
  return nullptr;
}

// The sums over the runs of k that a split product left in part[run][t][n], added in the order of the runs, go through
// the epilogue.  A thread takes four consecutive n of one token.
template <typename T, int EPI>
__global__ __launch_bounds__(256) void split_sum_kernel(const float* __restrict__ part, int runs, long long run_stride,
                                                        void* __restrict__ Y, int ldy, int N, int Tn) {
  const int n4 = (N + 3) / 4;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)Tn * n4) return;
  const int t = (int)(idx / n4), n = (int)(idx % n4) * 4;
  const float* p = part + (size_t)t * N + n;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if ((N & 3) == 0) {
    // eight runs at a time, all loads of a round on their way before the first sum (the last run stands in for those
    // beyond it, and is not added twice)
    for (int r0 = 0; r0 < runs; r0 += 8) {
      float4 x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = *(const float4*)(p + (size_t)(r0 + i < runs ? r0 + i : runs - 1) * run_stride);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (r0 + i < runs) {
          v[0] += x[i].x;
          v[1] += x[i].y;
          v[2] += x[i].z;
          v[3] += x[i].w;
        }
    }
  } else {
    for (int r = 0; r < runs; ++r)
      for (int e = 0; e < 4 && n + e < N; ++e) v[e] += p[(size_t)r * run_stride + e];
  }
  epilogue4<T, EPI>(Y, ldy, N, t, n, v[0], v[1], v[2], v[3]);
}

// The same sum for a product that adds into the float32 residual stream, one block per token, which then also leaves
// rmsnorm(new row) * norm_w in `normed` (run dtype): the norm that the next part would otherwise run as a kernel of
// its own (out = x * (1 / sqrt(sum(x^2)/N + eps)) * w, as rmsnorm.hip).  N is a multiple of 4, at most 1024 * NCH.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void split_sum_norm_kernel(const float* __restrict__ part, int runs, long long run_stride,
                                                             float* __restrict__ Y, int ldy, int N,
                                                             const float* __restrict__ norm_w, float eps, T* __restrict__ normed,
                                                             int ldn) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* p = part + (size_t)t * N;
  float* y = Y + (size_t)t * ldy;
  float4 row[NCH];
  float ss = 0.f;
  // the first eight runs of every piece of the row and the old values are all asked for before anything is added:
  // one trip to memory for the whole row (the last run stands in for those beyond it, and is not added twice)
  float4 old[NCH], x[NCH][8], nw[NCH];        // (the norm's weights too: asked for after the sum they would be a second trip)
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int n = (c * 256 + threadIdx.x) * 4;
    const int nn = n < N ? n : 0;
    old[c] = *(const float4*)(y + nn);
    nw[c] = *(const float4*)(norm_w + nn);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[c][i] = *(const float4*)(p + nn + (size_t)(i < runs ? i : runs - 1) * run_stride);
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int n = (c * 256 + threadIdx.x) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (n < N) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i < runs) {
          v.x += x[c][i].x;
          v.y += x[c][i].y;
          v.z += x[c][i].z;
          v.w += x[c][i].w;
        }
      for (int r = 8; r < runs; ++r) {
        const float4 more = *(const float4*)(p + n + (size_t)r * run_stride);
        v.x += more.x;
        v.y += more.y;
        v.z += more.z;
        v.w += more.w;
      }
      v.x += old[c].x;
      v.y += old[c].y;
      v.z += old[c].z;
      v.w += old[c].w;
      *(float4*)(y + n) = v;
      ss += v.x * v.x;
      ss += v.y * v.y;
      ss += v.z * v.z;
      ss += v.w * v.w;
    }
    row[c] = v;
  }
  ss = block_sum<4>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)N + eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int n = (c * 256 + threadIdx.x) * 4;
    if (n < N) {
      const float4 w = nw[c];
      T* o = normed + (size_t)t * ldn + n;
      Elem<T>::store(o, row[c].x * scale * w.x);
      Elem<T>::store(o + 1, row[c].y * scale * w.y);
      Elem<T>::store(o + 2, row[c].z * scale * w.z);
      Elem<T>::store(o + 3, row[c].w * scale * w.w);
    }
  }
}

// Few rows of X and few rows of W leave a chip of 256 compute units idle unless k is shared out as well: the runs of
// k go to blocks of their own (64x64 tiles), and split_sum_kernel adds their sums in a fixed order.
template <typename T, int EPI, int BN = 64, int BT = 64, int WN = 2, int WT = 2, int NS = 4>
static const char* launch_split(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int splits,
                                float* part, hipStream_t stream) {
  const long long plane = (long long)Tn * N;
  const char* err = launch_direct<T, BN, BT, WN, WT, NS, EPI_STORE_F32>(W, X, part, N, Tn, K, ldw, ldx, N, stream, splits, plane);
  if (err) return err;
  const int nk_all = K / (int)(128 / sizeof(T)), nk_split = (nk_all + splits - 1) / splits;
  const int runs = (nk_all + nk_split - 1) / nk_split;
  const long long threads = (long long)Tn * ((N + 3) / 4);
  hipLaunchKernelGGL((split_sum_kernel<T, EPI>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, part, runs, plane, Y,
                     ldy, N, Tn);
  return nullptr;
}

// What gemm_direct_kernel asks of a product: whole 128-byte pieces along k, and row offsets within a tile that fit 32 bits.
static bool direct_takes(int K, int ldw, int ldx, size_t elem) {
  return K % (int)(128 / elem) == 0 && (size_t)256 * ldw * elem < (1ull << 32) && (size_t)256 * ldx * elem < (1ull << 32);
}

template <typename T, int BN, int BT, int WN, int WT, int EPI>
static const char* launch_tiled(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                                hipStream_t stream) {
  const int tiles_t = (Tn + BT - 1) / BT, tiles_n = (N + BN - 1) / BN;
  constexpr int smem = 2 * (BN + BT) * GEMM_ROWB;
  auto kernel = gemm_kernel<T, BN, BT, WN, WT, EPI>;
  static bool raised = false;      // more than 64 KB of LDS has to be asked for once per kernel
  if (smem > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) DLGO_FAIL("gemm: cannot get %d bytes of LDS: %s", smem, hipGetErrorString(e));
    raised = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_t * tiles_n)), dim3(WN * WT * WAVE), smem, stream, (const T*)W, (const T*)X, Y,
                     N, Tn, K, ldw, ldx, ldy, tiles_t);
  return nullptr;
}

// In how many runs a product shares its k tiles out when the choice is the kernel's (64x64 tiles).  Few rows of X and
// few tiles of output: a block for every compute unit, of at least eight k tiles.  More rows (a short prompt) and a long
// inner size: about two blocks a unit, at most four runs.  (Measured on the shapes of 1B, 3B and 8B Llamas.)
static int auto_splits(int N, int Tn, int nk_all, long long part_elems) {
  const long small = (long)((N + 63) / 64) * ((Tn + 63) / 64);
  int splits = 1;
  if (Tn <= 128) {
    if (small <= 64 && nk_all >= 32) {
      splits = (int)(256 / small);
      if (splits > nk_all / 8) splits = nk_all / 8;
    } else if (small <= 128 && nk_all >= 32) {
      // half the units would idle otherwise: two runs, or with one tile of rows up to four, as many as make the rounds
      // of 256 blocks times a block's k tiles least (more runs where that is equal: two blocks share a unit well)
      long best = 0;
      for (int s = 2; s <= (Tn <= 64 ? 4 : 2); ++s) {
        const long cost = ((small * s + 255) / 256) * ((nk_all + s - 1) / s);
        if (s == 2 || cost <= best) { best = cost; splits = s; }
      }
    }
  } else if (small <= 256 && nk_all >= 128) {
    splits = (int)(512 / small);
    if (splits > 4) splits = 4;
  }
  while (splits > 1 && (long long)splits * Tn * N > part_elems) --splits;
  return splits;
}

// Which of the kernels that load straight into LDS a product gets when the choice is the library's (20 = 256x256, 21 =
// 128x128 with two blocks a unit, 22 = 128x128 deeper, 23 = 64x64).  Few rows of X: the weights stream through small
// tiles, and so does any product of at most two small tiles a compute unit.  Else the large tile when it fills the
// chip; else two blocks of 128x128 on a unit when there are that many; else one, deeper.  (Measured on the shapes of a
// 1B Llama.)
static int direct_kind(int N, int Tn) {
  const long b256 = (long)((N + 255) / 256) * ((Tn + 255) / 256);
  const long big = (long)((N + 127) / 128) * ((Tn + 127) / 128);
  const long small = (long)((N + 63) / 64) * ((Tn + 63) / 64);
  if (Tn <= 64) return 23;
  if (Tn <= 128) return N >= 32768 ? 21 : 23;
  if (small <= 512) return 23;
  return b256 >= 192 ? 20 : (big > 256 ? 21 : 22);
}

template <typename T, int EPI, int NORM>
static const char* launch_direct_norm(int kind, const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy,
                                      hipStream_t stream, const TileNorm& tn) {
  if (kind == 20) return launch_direct<T, 256, 256, 4, 4, 2, EPI, NORM>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, 1, 0, tn);
  if (kind == 21) return launch_direct<T, 128, 128, 2, 4, 2, EPI, NORM>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, 1, 0, tn);
  if (kind == 22) return launch_direct<T, 128, 128, 4, 4, 3, EPI, NORM>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, 1, 0, tn);
  return launch_direct<T, 64, 64, 2, 2, 4, EPI, NORM>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, 1, 0, tn);
}

template <typename T, int EPI>
static const char* dispatch(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int force,
                            int splits, float* part, long long part_elems, hipStream_t stream) {
  // force: 0 = choose, 2 = 128x128 tiles, 3 = 64x64, 4 = 32x32, 12 = 256x256 with 8 waves, 14 = 64x128; direct loads
  // into LDS: 20 = 256x256 with 16 waves, 21 = 128x128 with 8 waves and two blocks on a compute unit, 22 = 128x128
  // with 16 waves and three stages, 23 = 64x64 with four stages.
  // splits: 0 = choose, 1 = every block sums the whole of k, more = k in that many runs (64x64 tiles; needs part)
  int kind = force;
  const bool direct = direct_takes(K, ldw, ldx, sizeof(T));
  if ((kind >= 20 || splits > 1) && !direct) DLGO_FAIL("gemm: kernel %d needs K %% %d == 0, got K=%d", kind, (int)(128 / sizeof(T)), K);
  const int nk_all = K / (int)(128 / sizeof(T));
  if (splits == 0) splits = kind == 0 && direct && part ? auto_splits(N, Tn, nk_all, part_elems) : 1;
  if (splits > 1) {
    DLGO_REQUIRE(kind == 0 || kind == 23, "gemm: k is split for the 64x64 tiles only, not kernel %d", kind);
    DLGO_REQUIRE(part && (long long)splits * Tn * N <= part_elems && ((uintptr_t)part & 15) == 0,
                 "gemm: %d runs of k need %lld floats of scratch, got %lld", splits, (long long)splits * Tn * N, part_elems);
    DLGO_REQUIRE(splits <= nk_all, "gemm: %d runs of k, but only %d tiles", splits, nk_all);
    return launch_split<T, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, splits, part, stream);
  }
  if (kind == 0 && direct) kind = direct_kind(N, Tn);
  if (kind == 23) return launch_direct<T, 64, 64, 2, 2, 4, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 20) return launch_direct<T, 256, 256, 4, 4, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 21) return launch_direct<T, 128, 128, 2, 4, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 22) return launch_direct<T, 128, 128, 4, 4, 3, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 0) {
    const long b256 = (long)((N + 255) / 256) * ((Tn + 255) / 256);
    const long big = (long)((N + 127) / 128) * ((Tn + 127) / 128);
    const long mid = (long)((N + 63) / 64) * ((Tn + 63) / 64);
    const long tall = (long)((N + 63) / 64) * ((Tn + 127) / 128);
    // the largest tile that still gives every compute unit a block, and two where one block would leave a SIMD one wave
    kind = b256 >= 256 ? 12 : (big >= 512 ? 2 : (tall >= 256 ? 14 : (big >= 256 ? 2 : (mid >= 256 ? 3 : 4))));
  }
  if (kind == 14) return launch_tiled<T, 64, 128, 2, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 12) return launch_tiled<T, 256, 256, 2, 4, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 2) return launch_tiled<T, 128, 128, 2, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  if (kind == 3) return launch_tiled<T, 64, 64, 2, 2, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
  return launch_tiled<T, 32, 32, 1, 1, EPI>(W, X, Y, N, Tn, K, ldw, ldx, ldy, stream);
}

template <typename T>
static const char* by_epilogue(const void* W, const void* X, void* Y, int N, int Tn, int K, int ldw, int ldx, int ldy, int epi,
                               int force, int splits, float* part, long long part_elems, hipStream_t stream) {
  switch (epi) {
    case EPI_STORE: return dispatch<T, EPI_STORE>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, splits, part, part_elems, stream);
    case EPI_ACCUM_F32: return dispatch<T, EPI_ACCUM_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, splits, part, part_elems, stream);
    case EPI_SWIGLU: return dispatch<T, EPI_SWIGLU>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, splits, part, part_elems, stream);
    case EPI_STORE_F32: return dispatch<T, EPI_STORE_F32>(W, X, Y, N, Tn, K, ldw, ldx, ldy, force, splits, part, part_elems, stream);
    default: DLGO_FAIL("gemm: unknown epilogue %d", epi);
  }
}

// Y[t, n] (epilogue) = sum_k X[t, k] W[n, k].  ldy counts elements of Y's own type; for the SwiGLU epilogue Y has N/2 columns.
// part (may be null): part_elems floats of scratch for products whose k is split over several blocks.
extern "C" const char* dlgo_gemm(const void* W, const void* X, void* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                 int ldy, int epilogue, int force_kind, int splits, float* part, long long part_elems,
                                 hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0, "gemm: bad sizes N=%d T=%d K=%d", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(K % epc == 0, "gemm: inner size %d must be a multiple of %d for 16-byte loads", K, epc);
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ldw >= K && ldx >= K, "gemm: row strides (%d, %d) must be multiples of %d and at least K", ldw, ldx, epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0, "gemm: W and X must be 16-byte aligned");
  DLGO_REQUIRE(((uintptr_t)Y & 3) == 0 || (dtype == DLGO_DTYPE_BF16 && ((uintptr_t)Y & 1) == 0), "gemm: Y must be aligned to its elements");
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm: ldy %d shorter than N %d", ldy, N);
  DLGO_REQUIRE(splits >= 0 && part_elems >= 0, "gemm: bad split %d", splits);
  DLGO_REQUIRE(force_kind == 0 || (force_kind >= 2 && force_kind <= 4) || force_kind == 12 || force_kind == 14 ||
                   (force_kind >= 20 && force_kind <= 23),
               "gemm: unknown kernel choice %d", force_kind);
  if (Tn == 0) return nullptr;
  const char* err = by_epilogue<elem_t>(W, X, Y, N, Tn, K, ldw, ldx, ldy, epilogue, force_kind, splits, part, part_elems, stream);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm");
  return nullptr;
}

// The number of runs dlgo_gemm would share k out in for this product, left to choose (1: it would not split).
extern "C" int dlgo_gemm_auto_splits(int dtype, int N, int Tn, int K, int ldw, int ldx, long long part_elems) {
  const size_t elem = dtype == DLGO_DTYPE_F32 ? 4 : 2;
  if (N <= 0 || Tn <= 0 || K <= 0 || !direct_takes(K, ldw, ldx, elem)) return 1;
  return auto_splits(N, Tn, K / (int)(128 / elem), part_elems);
}

// The runs alone: part[r][t][n] = sum over run r of k of X[t, k] W[n, k], r < the returned *runs (planes of Tn * N floats, one
// after the other).  For a caller whose next kernel adds the runs up as it reads them.
extern "C" const char* dlgo_gemm_parts(const void* W, const void* X, int dtype, int N, int Tn, int K, int ldw, int ldx, int splits,
                                       float* part, long long part_elems, int* runs, hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0 && runs, "gemm: bad sizes N=%d T=%d K=%d", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(direct_takes(K, ldw, ldx, sizeof(elem_t)), "gemm: a split product needs K %% %d == 0, got K=%d", 8 * epc, K);
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ldw >= K && ldx >= K, "gemm: row strides (%d, %d) must be multiples of %d and at least K", ldw, ldx, epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)part & 15) == 0, "gemm: W, X and the scratch must be 16-byte aligned");
  const int nk_all = K / (int)(128 / sizeof(elem_t));
  DLGO_REQUIRE(splits > 1 && splits <= nk_all, "gemm: %d runs of k with %d tiles", splits, nk_all);
  DLGO_REQUIRE(part && (long long)splits * Tn * N <= part_elems, "gemm: %d runs of k need %lld floats of scratch, got %lld", splits,
               (long long)splits * Tn * N, part_elems);
  const int nk_split = (nk_all + splits - 1) / splits;
  *runs = (nk_all + nk_split - 1) / nk_split;
  if (Tn == 0) return nullptr;
  const char* err = launch_direct<elem_t, 64, 64, 2, 2, 4, EPI_STORE_F32>(W, X, part, N, Tn, K, ldw, ldx, N, stream, splits, (long long)Tn * N);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_parts");
  return nullptr;
}

// Y += X W^T with k shared out in `splits` runs (> 1), and normed = rmsnorm(Y) * norm_w of the new rows beside it.
extern "C" const char* dlgo_gemm_accum_norm(const void* W, const void* X, float* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                            int ldy, int splits, float* part, long long part_elems, const float* norm_w, float eps,
                                            void* normed, int ldn, hipStream_t stream) {
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0, "gemm: bad sizes N=%d T=%d K=%d", N, Tn, K);
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(direct_takes(K, ldw, ldx, sizeof(elem_t)), "gemm: a split product needs K %% %d == 0, got K=%d", 8 * epc, K);
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ldw >= K && ldx >= K, "gemm: row strides (%d, %d) must be multiples of %d and at least K", ldw, ldx, epc);
  DLGO_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0, "gemm: W and X must be 16-byte aligned");
  DLGO_REQUIRE(N % 4 == 0 && N <= 8192 && ldy % 4 == 0 && ldy >= N && ldn >= N, "gemm: the sum with a norm takes N %% 4 == 0 up to 8192, got %d", N);
  DLGO_REQUIRE(((uintptr_t)Y & 15) == 0 && ((uintptr_t)norm_w & 15) == 0 && ((uintptr_t)part & 15) == 0, "gemm: Y, the norm weight and the scratch must be 16-byte aligned");
  DLGO_REQUIRE(eps > 0.f, "gemm: eps must be positive");
  const int nk_all = K / (int)(128 / sizeof(elem_t));
  DLGO_REQUIRE(splits > 1 && splits <= nk_all, "gemm: %d runs of k with %d tiles", splits, nk_all);
  DLGO_REQUIRE(part && (long long)splits * Tn * N <= part_elems, "gemm: %d runs of k need %lld floats of scratch, got %lld", splits,
               (long long)splits * Tn * N, part_elems);
  if (Tn == 0) return nullptr;
  const long long plane = (long long)Tn * N;
  const char* err = launch_direct<elem_t, 64, 64, 2, 2, 4, EPI_STORE_F32>(W, X, part, N, Tn, K, ldw, ldx, N, stream, splits, plane);
  if (err) return err;
  const int nk_split = (nk_all + splits - 1) / splits, runs = (nk_all + nk_split - 1) / nk_split;
#define SUM_NORM(C_)                                                                                                              \
  hipLaunchKernelGGL((split_sum_norm_kernel<elem_t, C_>), dim3((unsigned)Tn), dim3(256), 0, stream, part, runs, plane, Y, ldy, N, \
                     norm_w, eps, (elem_t*)normed, ldn)
  if (N <= 1024) SUM_NORM(1);
  else if (N <= 2048) SUM_NORM(2);
  else if (N <= 4096) SUM_NORM(4);
  else SUM_NORM(8);
#undef SUM_NORM
  DLGO_LAUNCH_CHECK("gemm_accum_norm");
  return nullptr;
}

// Whether the two entry points below take a product: the tiles that load straight into LDS, every block summing the
// whole of k (with part_elems floats of scratch at hand dlgo_gemm might share k out instead: then not).  role 1: the
// product that leaves the norm (N a multiple of 32, up to 8192); role 2: the one that applies it.
extern "C" int dlgo_gemm_tile_norm_takes(int dtype, int N, int Tn, int K, int ldw, int ldx, int role, long long part_elems) {
  const size_t elem = dtype == DLGO_DTYPE_F32 ? 4 : 2;
  if (dtype != DLGO_ELEM || N <= 0 || Tn <= 0 || K <= 0 || !direct_takes(K, ldw, ldx, elem)) return 0;
  if (auto_splits(N, Tn, K / (int)(128 / elem), part_elems) != 1) return 0;
  if (role == 1) return N % 32 == 0 && N <= 8192 ? 1 : 0;
  return role == 2 ? 1 : 0;
}

// residual [T, N] (float32) += X W^T, and for the RMSNorm that follows: unscaled [T, N] (run dtype) = new residual * norm_w,
// parts [T, N / 32] = each 32 columns' share of every row's sum of squares (*n_parts = N / 32).  The consumer is
// dlgo_gemm_tile_scaled (or gemm_rows.hip's dlgo_gemm_rows_scaled) with these parts.
extern "C" const char* dlgo_gemm_tile_leave(const void* W, const void* X, float* residual, int dtype, int N, int Tn, int K, int ldw,
                                            int ldx, int ldy, const float* norm_w, void* unscaled, int ld_unscaled, float* parts,
                                            long long parts_elems, int* n_parts, hipStream_t stream) {
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0 && ldw >= K && ldx >= K && ldy >= N && ld_unscaled >= N, "gemm_tile_leave: bad sizes");
  DLGO_REQUIRE(direct_takes(K, ldw, ldx, sizeof(elem_t)), "gemm_tile_leave: K must be a whole number of 128-byte pieces, got %d", K);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0,
               "gemm_tile_leave: W and X must be 16-byte aligned with row strides that keep them so");
  DLGO_REQUIRE(N % 32 == 0 && N <= 8192 && ldy % 4 == 0 && ld_unscaled % 4 == 0, "gemm_tile_leave: N a multiple of 32 up to 8192, got %d", N);
  DLGO_REQUIRE(residual && norm_w && unscaled && parts && n_parts && ((uintptr_t)residual & 15) == 0 && ((uintptr_t)norm_w & 15) == 0 &&
                   ((uintptr_t)unscaled & 7) == 0 && parts_elems >= (long long)Tn * (N / 32),
               "gemm_tile_leave: missing or misaligned operand, or scratch too small");
  *n_parts = N / 32;
  if (Tn == 0) return nullptr;
  const TileNorm tn{norm_w, unscaled, ld_unscaled, parts, N / 32, 0, 0.f};
  const char* err = launch_direct_norm<elem_t, EPI_ACCUM_F32, 1>(direct_kind(N, Tn), W, X, residual, N, Tn, K, ldw, ldx, ldy, stream, tn);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_tile_leave");
  return nullptr;
}

// Y (epilogue)= scale[t] * (X W^T), X being rows left unscaled with the shares of their sums of squares in parts:
// scale[t] = 1 / sqrt(sum of the row's parts / width + eps).  Epilogues: store and SwiGLU.
extern "C" const char* dlgo_gemm_tile_scaled(const void* W, const void* X, void* Y, int dtype, int N, int Tn, int K, int ldw, int ldx,
                                             int ldy, int epilogue, const float* parts, int n_parts, int width, float eps,
                                             hipStream_t stream) {
  DLGO_REQUIRE(dtype == DLGO_ELEM, "gemm: this library is built for dtype code %d, got %d", DLGO_ELEM, dtype);
  DLGO_REQUIRE(N > 0 && Tn >= 0 && K > 0 && ldw >= K && ldx >= K, "gemm_tile_scaled: bad sizes");
  DLGO_REQUIRE(direct_takes(K, ldw, ldx, sizeof(elem_t)), "gemm_tile_scaled: K must be a whole number of 128-byte pieces, got %d", K);
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  DLGO_REQUIRE(ldw % epc == 0 && ldx % epc == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)X & 15) == 0,
               "gemm_tile_scaled: W and X must be 16-byte aligned with row strides that keep them so");
  DLGO_REQUIRE(parts && n_parts > 0 && width > 0 && eps > 0.f, "gemm_tile_scaled: parts, their number, the width and eps");
  DLGO_REQUIRE(epilogue == EPI_STORE || epilogue == EPI_SWIGLU, "gemm_tile_scaled: epilogues store and SwiGLU, got %d", epilogue);
  DLGO_REQUIRE(epilogue != EPI_SWIGLU || (N % 2 == 0 && ldy >= N / 2), "gemm: SwiGLU epilogue needs an even N and ldy >= N/2");
  DLGO_REQUIRE(epilogue == EPI_SWIGLU || ldy >= N, "gemm: ldy %d shorter than N %d", ldy, N);
  if (Tn == 0) return nullptr;
  const TileNorm tn{nullptr, nullptr, 0, const_cast<float*>(parts), n_parts, width, eps};
  const int kind = direct_kind(N, Tn);
  const char* err = epilogue == EPI_STORE
                        ? launch_direct_norm<elem_t, EPI_STORE, 2>(kind, W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, tn)
                        : launch_direct_norm<elem_t, EPI_SWIGLU, 2>(kind, W, X, Y, N, Tn, K, ldw, ldx, ldy, stream, tn);
  if (err) return err;
  DLGO_LAUNCH_CHECK("gemm_tile_scaled");
  return nullptr;
}

#if DLGO_ELEM == DLGO_DTYPE_F32
#include "exact_end.h"
#endif

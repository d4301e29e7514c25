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
// everything here is float32 arithmetic whatever the storage type: no approximation can be named (exact_begin.h)
#include "exact_begin.h"

#define PAGE 64

template <typename T>
__global__ __launch_bounds__(WAVE) void rope_kv_kernel(T* __restrict__ qkv, int ld, int n_heads, int n_kv, int hd, int rot,
                                                       int interleaved, const float* __restrict__ cos_t,
                                                       const float* __restrict__ sin_t, const int32_t* __restrict__ positions,
                                                       const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
                                                       const int32_t* __restrict__ page_table, int max_pages,
                                                       T* __restrict__ cache, long long page_stride, long long v_off,
                                                       int write_kv, int by_row) {
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
    const int row = by_row ? t : slots[tok_seq[t]];   // the table's rows: in the order of the step's rows, or by slot
    const int page = page_table[(size_t)row * max_pages + pos / PAGE];
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
      const float y0 = rotated_lo(x0, x1, cs, sn);
      const float y1 = rotated_hi(x0, x1, cs, sn);
      x0 = y0;
      x1 = y1;
    }
    Elem<T>::store(dst + i0, x0);
    Elem<T>::store(dst + i1, x1);
  }
  if (is_k)   // the part of the head beyond the rotated width is copied
    for (int i = rot + lane; i < hd; i += WAVE) kdst[i] = src[i];
}

// The same work in 16-byte pieces, one thread per piece of a token's [q | k | v] row, for rotated widths whose halves
// are whole pieces (every model of a usual shape): a piece is read once, rotated against its partner piece, and
// written once (queries in place, keys as one 16-byte store, values scattered into their transposed page).
template <typename T> struct Piece;
template <> struct Piece<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void load(const float* p, float* f) { *(float4*)f = *(const float4*)p; }
  static __device__ __forceinline__ void store(float* p, const float* f) { *(float4*)p = *(const float4*)f; }
};
template <> struct Piece<bf16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* f) {
    const uint4 u = *(const uint4*)p;
    f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
    f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
    f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
    f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float* f) {
    uint4 u;
    u.x = (uint32_t)f32_to_bf16(f[0]) | ((uint32_t)f32_to_bf16(f[1]) << 16);
    u.y = (uint32_t)f32_to_bf16(f[2]) | ((uint32_t)f32_to_bf16(f[3]) << 16);
    u.z = (uint32_t)f32_to_bf16(f[4]) | ((uint32_t)f32_to_bf16(f[5]) << 16);
    u.w = (uint32_t)f32_to_bf16(f[6]) | ((uint32_t)f32_to_bf16(f[7]) << 16);
    *(uint4*)p = u;
  }
};

// The E elements at column `col` of row t: from the rows themselves, or, where the product that made the rows left the
// runs of its inner sum unsummed (n_parts planes of float32, `plane` apart, rows of part_ld), their sum in run order.
template <typename T, bool SUMS>
static __device__ __forceinline__ void load_piece(const T* __restrict__ qkv, int ld, const float* __restrict__ part, int n_parts,
                                                  long long plane, int part_ld, int t, int col, float* x) {
  constexpr int E = Piece<T>::E;
  if constexpr (!SUMS) {
    Piece<T>::load(qkv + (size_t)t * ld + col, x);
    return;
  } else {
  const float* p = part + (size_t)t * part_ld + col;
#pragma unroll
  for (int e = 0; e < E; e += 4) *(float4*)(x + e) = *(const float4*)(p + e);
  for (int r = 1; r < n_parts; ++r) {
    p += plane;
#pragma unroll
    for (int e = 0; e < E; e += 4) {
      const float4 v = *(const float4*)(p + e);
      x[e] += v.x;
      x[e + 1] += v.y;
      x[e + 2] += v.z;
      x[e + 3] += v.w;
    }
  }
  }
}

// Holds a loaded piece to this place of the program: the compiler may not move its load below (it would otherwise sink a
// load past a wait for another, into the branch that uses it, and so make two trips to memory of one).
template <int E>
static __device__ __forceinline__ void asked_by_here(const float* x) {
#pragma unroll
  for (int e = 0; e < E; ++e) asm volatile("" ::"v"(x[e]));
}

// The page that holds position pos of row t's sequence.  BYROW: the table's rows are in the order of the step's rows (a
// step of single tokens, whose caller keeps such a table); else by slot, through the row's sequence and its slot.
template <bool BYROW>
static __device__ __forceinline__ int page_of(int t, int pos, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
                                              const int32_t* __restrict__ page_table, int max_pages) {
  if constexpr (BYROW) return page_table[(size_t)t * max_pages + pos / PAGE];
  else return page_table[(size_t)slots[tok_seq[t]] * max_pages + pos / PAGE];
}

// WRITES: keys and values go into the cache; SUMS: the rows come as unsummed runs; BYROW: see page_of.  All are known at
// the launch, and as template arguments they leave no load under a condition, which the compiler would make wait for
// every load before it: a thread asks for its piece, its partner piece and its position together, then for the page and
// the angles, and stores.  The blocks of the values come first in the grid: their way to the page is the longest.
template <typename T, bool WRITES, bool SUMS, bool BYROW>
__global__ __launch_bounds__(256) void rope_kv_pieces_kernel(T* __restrict__ qkv, int ld, int n_tokens, int n_heads, int n_kv, int hd,
                                                             int rot, int interleaved, const float* __restrict__ cos_t,
                                                             const float* __restrict__ sin_t,
                                                             const int32_t* __restrict__ positions,
                                                             const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ slots,
                                                             const int32_t* __restrict__ page_table, int max_pages,
                                                             T* __restrict__ cache, long long page_stride, long long v_off,
                                                             int value_blocks, const float* __restrict__ part, int n_parts,
                                                             long long plane, int part_ld, int single_tokens) {
  constexpr int E = Piece<T>::E;
  if (WRITES && (int)blockIdx.x < value_blocks && single_tokens) {
    // The values of a step of single tokens: every row belongs to another sequence, so nothing of the transposed page
    // rows is consecutive and a tile would gain nothing: a thread stores the piece it read, element by element.
    const int per_head = hd / E;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)n_tokens * n_kv * per_head) return;
    const int t = (int)(idx / (n_kv * per_head)), c = (int)(idx % (n_kv * per_head));
    const int kvh = c / per_head, d0 = (c % per_head) * E;
    float x[E];
    load_piece<T, SUMS>(qkv, ld, part, n_parts, plane, part_ld, t, (n_heads + n_kv + kvh) * hd + d0, x);
    const int pos = positions[t];
    const int page = page_of<BYROW>(t, pos, tok_seq, slots, page_table, max_pages);
    asked_by_here<E>(x);
    if (page < 0) return;
    T* vcol = cache + v_off + (size_t)page * page_stride + ((size_t)kvh * hd + d0) * PAGE + pos % PAGE;
#pragma unroll
    for (int e = 0; e < E; ++e) Elem<T>::store(vcol + (size_t)e * PAGE, x[e]);
    return;
  }
  if (WRITES && (int)blockIdx.x < value_blocks) {
    // The values.  A page keeps them transposed ([head size][token]), so a thread that stored its own piece would write
    // single elements a page row apart.  Instead a block takes 64 consecutive rows of the step, one kv head and up to 64
    // of its dimensions, turns the tile through LDS, and stores with its lanes along the tokens: where the rows are
    // consecutive tokens of a sequence, a wave writes a run of a page row at a time.
    __shared__ T tile[64][66];
    const int per_tok_tile = (hd + 63) / 64;
    const int b = blockIdx.x;
    const int dpart = b % per_tok_tile, kvh = (b / per_tok_tile) % n_kv, t0 = (b / per_tok_tile / n_kv) * 64;
    const int dbase = dpart * 64, db = hd - dbase < 64 ? hd - dbase : 64;
    const int ppr = db / E;                                  // pieces per row of the tile
    // the page of the row that this thread will store, asked for before the tile (a row past the end asks the last row's)
    const int tk = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int t = t0 + tk < n_tokens ? t0 + tk : n_tokens - 1;
    const int pos = positions[t];
    const int page = page_of<BYROW>(t, pos, tok_seq, slots, page_table, max_pages);
    for (int c = threadIdx.x; c < 64 * ppr; c += 256) {
      const int rk = c / ppr, pc = c % ppr;
      if (t0 + rk < n_tokens) {
        float x[E];
        load_piece<T, SUMS>(qkv, ld, part, n_parts, plane, part_ld, t0 + rk, (n_heads + n_kv + kvh) * hd + dbase + pc * E, x);
#pragma unroll
        for (int e = 0; e < E; ++e) Elem<T>::store(&tile[rk][pc * E + e], x[e]);
      }
    }
    __syncthreads();
    if (t0 + tk >= n_tokens || page < 0) return;
    T* vcol = cache + v_off + (size_t)page * page_stride + ((size_t)kvh * hd + dbase) * PAGE + pos % PAGE;
    for (int d = w; d < db; d += 4) vcol[(size_t)d * PAGE] = tile[tk][d];
    return;
  }
  const int per_head = hd / E;
  const int heads = n_heads + (WRITES ? n_kv : 0);          // queries and keys; the values have blocks of their own
  const int per_token = heads * per_head;
  const long long idx = (long long)((int)blockIdx.x - (WRITES ? value_blocks : 0)) * 256 + threadIdx.x;
  if (idx >= (long long)n_tokens * per_token) return;
  const int t = (int)(idx / per_token), c = (int)(idx % per_token);
  const int head = c / per_head, d0 = (c % per_head) * E;
  T* src = qkv + (size_t)t * ld + (size_t)head * hd;
  const bool is_q = head < n_heads;
  const bool rotates = cos_t && d0 < rot;
  const int half = rot / 2;
  const bool pairs_far = rotates && !interleaved;          // the partner is the piece half a rotated width on
  if (pairs_far && d0 >= half) return;                     // done by the thread of the partner piece
  float x[E], p[E];
  load_piece<T, SUMS>(qkv, ld, part, n_parts, plane, part_ld, t, head * hd + d0, x);
  load_piece<T, SUMS>(qkv, ld, part, n_parts, plane, part_ld, t, head * hd + d0 + (pairs_far ? half : 0), p);
  const int pos = positions[t];
  int page = 0;
  if constexpr (WRITES) page = page_of<BYROW>(t, pos, tok_seq, slots, page_table, max_pages);
  asked_by_here<E>(x);
  asked_by_here<E>(p);
  if (!rotates) {
    if (!is_q && page < 0) return;
    T* dst = is_q ? src : cache + (size_t)page * page_stride + ((size_t)(head - n_heads) * PAGE + pos % PAGE) * hd;
    if (!is_q || SUMS) Piece<T>::store(dst + d0, x);        // the part of a key beyond the rotated width is copied
    return;
  }
  // angles: for interleaved pairs the E/2 of this piece, else the E of its pair of pieces
  const float* cs = cos_t + (size_t)pos * half + (interleaved ? d0 / 2 : d0);
  const float* sn = sin_t + (size_t)pos * half + (interleaved ? d0 / 2 : d0);
  float c_[E], s_[E];
#pragma unroll
  for (int e = 0; e < E / 2; ++e) c_[e] = cs[e], s_[e] = sn[e];
  if (!interleaved) {
#pragma unroll
    for (int e = E / 2; e < E; ++e) c_[e] = cs[e], s_[e] = sn[e];
  }
  // where the rotated pieces go: queries in place, keys into their page
  if (!is_q && page < 0) return;
  T* dst = is_q ? src : cache + (size_t)page * page_stride + ((size_t)(head - n_heads) * PAGE + pos % PAGE) * hd;
  if (interleaved) {
    float y[E];
#pragma unroll
    for (int i = 0; i < E / 2; ++i) {
      y[2 * i] = rotated_lo(x[2 * i], x[2 * i + 1], c_[i], s_[i]);
      y[2 * i + 1] = rotated_hi(x[2 * i], x[2 * i + 1], c_[i], s_[i]);
    }
    Piece<T>::store(dst + d0, y);
  } else {
    // this thread owns the pieces at d0 and d0 + half: both were read before either is written
    float y0[E], y1[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
      y0[e] = rotated_lo(x[e], p[e], c_[e], s_[e]);
      y1[e] = rotated_hi(x[e], p[e], c_[e], s_[e]);
    }
    Piece<T>::store(dst + d0, y0);
    Piece<T>::store(dst + d0 + half, y1);
  }
}

extern "C" const char* dlgo_rope_kv(void* qkv, int dtype, int n_tokens, int ld, int n_heads, int n_kv, int hd, int rot,
                                    int interleaved, const float* cos_t, const float* sin_t, int table_rows,
                                    const int32_t* positions, const int32_t* tok_seq, const int32_t* slots,
                                    const int32_t* page_table, int max_pages, void* cache, long long page_stride,
                                    long long v_off, int write_kv, const float* part, int n_parts, long long plane, int part_ld,
                                    int single_tokens, int by_row, hipStream_t stream) {
  DLGO_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv >= 0 && hd > 0, "rope_kv: bad sizes");
  DLGO_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv: rotated width %d must be even and at most head_dim %d", rot, hd);
  DLGO_REQUIRE(ld >= (n_heads + 2 * n_kv) * hd, "rope_kv: row stride %d shorter than the heads it holds", ld);
  DLGO_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_kv: cos and sin tables come together");
  DLGO_REQUIRE(cos_t == nullptr || table_rows > 0, "rope_kv: empty rotation table");
  // by_row: page_table's rows are in the order of the step's rows (one token a sequence), not by slot
  DLGO_REQUIRE(!write_kv || (cache && page_table && (by_row || (slots && tok_seq)) && max_pages > 0), "rope_kv: cache arguments missing");
  if (n_tokens == 0) return nullptr;
  const int epc = dtype == DLGO_DTYPE_F32 ? 4 : 8;
  const bool pieces = hd % epc == 0 && rot % (2 * epc) == 0 && ld % epc == 0 && ((uintptr_t)qkv & 15) == 0 &&
                      (!write_kv || (((uintptr_t)cache & 15) == 0 && page_stride % epc == 0 && v_off % epc == 0));
  // part: the rows are still the n_parts unsummed runs of the product that makes them (float32 planes of rows of part_ld);
  // the kernel sums them as it reads, and writes the queries into qkv
  DLGO_REQUIRE(!part || (pieces && n_parts >= 1 && part_ld % 4 == 0 && part_ld >= (n_heads + (write_kv ? 2 * n_kv : 0)) * hd &&
                         plane >= (long long)n_tokens * part_ld && plane % 4 == 0 && ((uintptr_t)part & 15) == 0),
               "rope_kv: unsummed rows need whole 16-byte pieces (head size %d, rotated width %d) and aligned planes", hd, rot);
  if (pieces) {
    const long long items = (long long)n_tokens * (n_heads + (write_kv ? n_kv : 0)) * (hd / epc);
    const long long piece_blocks = (items + 255) / 256;
    // single_tokens: every row is a sequence of its own (a decode step); the values then go thread by thread
    const long long value_blocks = !write_kv ? 0
                                   : single_tokens ? ((long long)n_tokens * n_kv * (hd / epc) + 255) / 256
                                                   : (long long)((n_tokens + 63) / 64) * n_kv * ((hd + 63) / 64);
    DLGO_REQUIRE(piece_blocks + value_blocks < (1ll << 31), "rope_kv: too many rows at once");
    dim3 g((unsigned)(piece_blocks + value_blocks));
    const bool rows = by_row != 0;
#define DLGO_ROPE_PIECES(T, WRITES, SUMS, BYROW)                                                                               \
  hipLaunchKernelGGL((rope_kv_pieces_kernel<T, WRITES, SUMS, BYROW>), g, dim3(256), 0, stream, (T*)qkv, ld, n_tokens, n_heads,  \
                     n_kv, hd, rot, interleaved, cos_t, sin_t, positions, tok_seq, slots, page_table, max_pages, (T*)cache,    \
                     page_stride, v_off, (int)value_blocks, part, n_parts, plane, part_ld, single_tokens)
#define DLGO_ROPE_PIECES_OF(T)                                           \
  do {                                                                   \
    if (write_kv && part && rows) DLGO_ROPE_PIECES(T, true, true, true);      \
    else if (write_kv && part) DLGO_ROPE_PIECES(T, true, true, false);        \
    else if (write_kv && rows) DLGO_ROPE_PIECES(T, true, false, true);        \
    else if (write_kv) DLGO_ROPE_PIECES(T, true, false, false);               \
    else if (part) DLGO_ROPE_PIECES(T, false, true, false);                   \
    else DLGO_ROPE_PIECES(T, false, false, false);                            \
  } while (0)
    if (dtype == DLGO_DTYPE_F32) DLGO_ROPE_PIECES_OF(float);
    else if (dtype == DLGO_DTYPE_BF16) DLGO_ROPE_PIECES_OF(bf16_t);
    else DLGO_FAIL("rope_kv: unknown dtype code %d", dtype);
#undef DLGO_ROPE_PIECES_OF
#undef DLGO_ROPE_PIECES
    DLGO_LAUNCH_CHECK("rope_kv");
    return nullptr;
  }
  dim3 grid(n_tokens, n_heads + 2 * n_kv);
  if (dtype == DLGO_DTYPE_F32)
    hipLaunchKernelGGL(rope_kv_kernel<float>, grid, dim3(WAVE), 0, stream, (float*)qkv, ld, n_heads, n_kv, hd, rot, interleaved,
                       cos_t, sin_t, positions, tok_seq, slots, page_table, max_pages, (float*)cache, page_stride, v_off, write_kv, by_row);
  else if (dtype == DLGO_DTYPE_BF16)
    hipLaunchKernelGGL(rope_kv_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, (bf16_t*)qkv, ld, n_heads, n_kv, hd, rot, interleaved,
                       cos_t, sin_t, positions, tok_seq, slots, page_table, max_pages, (bf16_t*)cache, page_stride, v_off, write_kv, by_row);
  else
    DLGO_FAIL("rope_kv: unknown dtype code %d", dtype);
  DLGO_LAUNCH_CHECK("rope_kv");
  return nullptr;
}

#include "exact_end.h"

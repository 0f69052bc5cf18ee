// BLAST at 2 to 16 token rows as three launches: y = x V on the matrix cores, the rank-space mix, out = z U on the matrix cores.
// Low rank runs as BLAST with one output block and S = 1 (its middle launch adds the k-slices of x A), Monarch as two launches
// (its permutation is the store pattern of the first product) or, with input blocks deeper than 1024 rows, as three (the
// blocks are cut into slices; the middle launch adds them while it permutes).  A middle launch that only adds slices also
// carries workgroups that load the second product's factor into L2 (rows_prefetch).
//
// rows_product_kernel computes a batch of skinny products  out[bt] (M x N) = A[bt] (M x K) W[bt] (K x N),  M <= 16, with W
// row-major (the column index contiguous) - the layout of V (b, p, r) and of U (b, r, q).  A workgroup of eight waves owns
// all K rows of a chunk of up to 128 columns; each wave streams an eighth of the rows, so a lane has at most 32 16-byte
// loads, all issued before the first product (no ring, no branch around a load: rows past the end of the factor are out
// of the buffer's bounds and read as zero).  The matrix cores want, per lane, eight consecutive k of ONE column, and a
// 16-byte load delivers eight columns of one k.  Nothing is transposed: the lane loads eight rows, and the product with
// index e (0..7) takes element e of each of them (two byte-permutes per register pair) - the 16 column slots of that
// product are then the columns 8 n + e of the chunk, n = 0..15, which is only a naming of the accumulators.  The eight
// waves' partial sums meet in LDS, are added in wave order and leave as T.
//
// Why three launches and not the single-launch hand-over kernel: a kernel boundary on one stream costs about 1 us and
// what crosses it is ordinary cached memory, a hand-over inside a launch costs 1.5 us per hop, and at these row counts
// the mix is too much work to be redone by every slab of an output block (as the two-launch path for up to four rows
// does).  The number of column pieces per chunk is planned so that the chunks spread evenly over the compute units
// (a compute unit draws about 35 GB/s, so the bytes of the busiest one bound the launch).
#include <type_traits>
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
constexpr int DR_NT = 512;
constexpr int DR_WAVES = 8;
constexpr int DR_MAX_STEPS = 4;           // 32-row steps of a wave: 8 loads per lane each
constexpr int DR_MAX_M = 128;             // token rows: tiles of 16 over the same registers of weights
constexpr uint32_t DR_OOB = 0x80000000u;
}  // namespace

#ifdef BLR_TRACE
__device__ unsigned long long g_trace5[1024 * 16];
#define TR5(i) do { if (threadIdx.x == 0 && blockIdx.x < 512) g_trace5[(p.trace_base + blockIdx.x) * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR5(i) do {} while (0)
#endif

struct RowsParams {
  const void* A; int64_t lda, a_bs;       // A[m * lda + bt * a_bs + k]; rows m >= M read as zero
  uint32_t a_bytes;
  const void* W; int64_t w_bs;            // W[bt * w_bs + k * N + n]: T, int8 codes, or int4 codes two to a byte
  void* out; int64_t o_ms, o_bs, o_ns;    // out[m * o_ms + bt * o_bs + n * o_ns]
  const void* bias; int act;              // fused output stage (bias of T indexed like a row of out, or null; blr_act), applied to
                                          // the result rounded to T - what a separate elementwise kernel would see
  int ep;
  int out_f32;                            // the product is one slice of a reduction: out holds fp32 partial sums (plain row-major
                                          // store, no scales, no output stage) that the next launch adds in slice order
  const f16* scales;                      // codes: the product's column n of entry bt is multiplied by scales[bt * N + n]; else null
  int M, K, N;
  int kw;                                 // rows of a wave's share per round (a multiple of 32)
  int rounds;                             // passes of the eight waves over the rows
  int mtiles;                             // 16-row tiles of A and out (M <= 16: one); more than one only with rounds == 1: the
                                          // weights then stay in registers and every further tile costs products and a reduction
  int per; int64_t o_ls; FastDiv perdiv;  // per > 0: Monarch scatter - column c of entry bt goes to out[(c / per) * o_ls + m * o_ms + bt * per + c % per]
  int npc;                                // 16-byte column pieces of a chunk (1..16)
  FastDiv nch;                            // chunks per batch entry
  uint32_t xcd_span;                      // items per XCD when the grid is a multiple of 8, else 0 (plain order)
  int trace_base;
};

template <typename T> struct RowsMfma;
template <> struct RowsMfma<f16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct RowsMfma<bf16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// A lane's piece of one weight row: eight columns, as 16 bytes of T, 8 bytes of int8 codes or 4 bytes of int4 codes (low nibble
// first), and its expansion to eight packed T.  For f16 the codes go through the exponent trick: byte u (the code with its
// sign bit flipped) under the high byte 0x64 is the f16 number 1024 + u, and 1024 + u - 1152 = code, exactly.
template <typename T, int WB> struct RowsPiece;
template <typename T> struct RowsPiece<T, 16> {
  using raw_t = u32x4;
  static __device__ __forceinline__ raw_t load(__amdgpu_buffer_rsrc_t r, uint32_t off) { return ldw16(r, off, 0); }
  static __device__ __forceinline__ u32x4 expand(raw_t v) { return v; }
};
template <typename T, int WB> struct RowsCodes {
  // generic: through fp32 (exact for these small integers in either 16-bit type)
  static __device__ __forceinline__ u32x4 expand8(const int (&c)[8]) {
    typename TypeTraits<T>::vec8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = TypeTraits<T>::from_f32((float)c[e]);
    return __builtin_bit_cast(u32x4, v);
  }
};
template <typename T> struct RowsPiece<T, 8> {
  using raw_t = u32x2;
  static __device__ __forceinline__ raw_t load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 2));
  }
  static __device__ __forceinline__ u32x4 expand(raw_t v) {
    if constexpr (sizeof(T) == 2 && __is_same(T, f16)) {
      const f16x2 bias = {(f16)1152.0f, (f16)1152.0f};
      u32x4 o;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const uint32_t u = v[d] ^ 0x80808080u;
        const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u), hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
        o[2 * d] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, lo) - bias);
        o[2 * d + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, hi) - bias);
      }
      return o;
    } else {
      int c[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) c[e] = (int)(int8_t)((v[e >> 2] >> ((e & 3) * 8)) & 0xFF);
      return RowsCodes<T, 8>::expand8(c);
    }
  }
};
template <typename T> struct RowsPiece<T, 4> {
  using raw_t = uint32_t;
  static __device__ __forceinline__ raw_t load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 2);
  }
  static __device__ __forceinline__ u32x4 expand(raw_t v) {
    if constexpr (__is_same(T, f16)) {
      const f16x2 bias = {(f16)1032.0f, (f16)1032.0f};
      const uint32_t u = v ^ 0x88888888u, uh = u >> 4;
      u32x4 o;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // byte d of u holds the codes of columns 2d (low nibble) and 2d + 1 (high nibble)
        const uint32_t sel = 0x0C040C00u + (uint32_t)d * 0x00010001u;      // {0, uh.byte d, 0, u.byte d}
        const uint32_t pr = (__builtin_amdgcn_perm(uh, u, sel) & 0x000F000Fu) | 0x64006400u;
        o[d] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, pr) - bias);
      }
      return o;
    } else {
      int c[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) c[e] = ((int32_t)(v << (28 - 4 * e))) >> 28;
      return RowsCodes<T, 4>::expand8(c);
    }
  }
};

// NK: the factor is stored transposed, W[bt][n][k] with k contiguous (U of the bmm names, (b, q, r)).  A 16-byte load then is
// a lane's matrix-core operand as it stands: the lane of slot n and k-group g loads k .. k + 7 of column 16 cg + n for each of
// the chunk's column groups cg (p.npc of them, 16 columns each).
// MULTI: more than one tile of 16 token rows (a separate instantiation: the single-tile kernel carries none of the loop).
template <typename T, int STEPS, int WB, bool NK, bool MULTI>
__global__ __launch_bounds__(DR_NT) void rows_product_kernel(RowsParams p) {
  using Piece = RowsPiece<T, WB>;
  static_assert(!NK || WB == 16, "codes are stored (k, n)");
  __shared__ __attribute__((aligned(16))) float red[DR_WAVES * 16 * 128];
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
  TR5(0);
  // workgroup w runs on XCD w % 8: neighbouring chunks (which share cache lines when a chunk's row piece is not a whole
  // number of lines) go to one XCD, i.e. one L2
  const uint32_t item = p.xcd_span ? (blockIdx.x & 7u) * p.xcd_span + (blockIdx.x >> 3) : blockIdx.x;
  const uint32_t bt = fd_div(item, p.nch), ch = item - bt * p.nch.d;
  const int N = p.N, K = p.K;
  const int cw = p.npc * (NK ? 16 : 8);                  // columns of a chunk
  const int col0 = (int)ch * cw;                         // first column of the chunk
  const int colp = col0 + (NK ? n : n * 8);              // first column of this lane's pieces
  const bool live = NK ? true : (n < p.npc && colp < N);
  const __amdgpu_buffer_rsrc_t abuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.A), 0, p.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wb = wbuf(reinterpret_cast<const char*>(p.W) + (int64_t)bt * p.w_bs * WB / 8, (uint32_t)((int64_t)K * N * WB / 8));
  f32x4 acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
  // More than 8 waves x STEPS x 32 rows: the workgroup passes over the rows in rounds (the loads of a round are issued when
  // the products of the one before are done - one more trip to memory per extra round).
  u32x4 av[STEPS];
  typename Piece::raw_t wr[STEPS][8];
  auto products = [&]() {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if constexpr (NK) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = RowsMfma<T>::run(av[s], Piece::expand(wr[s][e]), acc[e]);
      } else {
        u32x4 wx[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) wx[t] = Piece::expand(wr[s][t]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
          u32x4 bv;
#pragma unroll
          for (int h = 0; h < 4; ++h) bv[h] = __builtin_amdgcn_perm(wx[2 * h + 1][e >> 1], wx[2 * h][e >> 1], sel);
          acc[e] = RowsMfma<T>::run(av[s], bv, acc[e]);
        }
      }
    }
  };
  for (int ro = 0; ro < p.rounds; ++ro) {
  const int kb = (ro * DR_WAVES + wv) * p.kw + 8 * g;    // first of this lane's eight k of step 0

  // activations: row n of A, the lane's eight k of every step (16 bytes each); weights: eight rows per step, the lane's
  // 16-byte piece of each.  Lanes without a row / without a column piece issue nothing (their registers stay undefined:
  // they only reach rows and columns of the product that are never stored), so a narrow chunk costs the load path
  // only what its live lanes fetch.
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    asm volatile("" : "=v"(av[s]));
#pragma unroll
    for (int t = 0; t < 8; ++t) asm volatile("" : "=v"(wr[s][t]));
  }
  if (n < p.M) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = kb + 32 * s;
      const uint32_t off = k < K ? (uint32_t)((int64_t)n * p.lda + (int64_t)bt * p.a_bs + k) * 2u : DR_OOB;
      av[s] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(abuf, off, 0, 0));
    }
  } else {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) av[s] = u32x4{0u, 0u, 0u, 0u};
  }
  if constexpr (NK) {
    // columns past the factor and k past K read as zero (offset out of the buffer's bounds); column groups past the chunk are
    // not asked for at all (a load costs its turn in the memory pipeline even with every lane out of bounds; their registers
    // stay undefined and only reach columns that are never stored)
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      if (t < p.npc) {
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          const int c = colp + 16 * t, k = kb + 32 * s;
          wr[s][t] = Piece::load(wb, (c < N && k < K) ? (uint32_t)(c * K + k) * 2u : DR_OOB);
        }
      }
    }
  } else if (live) {
    const uint32_t wbase = (uint32_t)(kb * N + colp) * (uint32_t)WB / 8u;
    const uint32_t rowb = (uint32_t)N * (uint32_t)WB / 8u;
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < 8; ++t) wr[s][t] = Piece::load(wb, wbase + (uint32_t)(32 * s + t) * rowb);
  }

  TR5(1);
  products();
  }  // rounds
  TR5(2);
  // More than 16 rows (one round only): the weights stay in the registers; per further tile of 16 rows the activations are
  // fetched (asked for before the reduction of the tile before, so that they arrive under it), multiplied and reduced.
  for (int mt = 0;; ++mt) {
  const int mrow0 = mt * 16;
  const bool more = MULTI && mt + 1 < p.mtiles;
  u32x4 avn[STEPS];
  if (MULTI && more) {
    const int row = mrow0 + 16 + n, kb = wv * p.kw + 8 * g;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = kb + 32 * s;
      const uint32_t off = (row < p.M && k < K) ? (uint32_t)((int64_t)row * p.lda + (int64_t)bt * p.a_bs + k) * 2u : DR_OOB;
      avn[s] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(abuf, off, 0, 0));
    }
  }
  if constexpr (NK) {
    // acc[e][t] is row 4 g + t, column col0 + 16 e + n
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) red[((wv * 16 + 4 * g + t) * 128) + 16 * e + n] = acc[e][t];
  } else {
    // acc[e][t] is row 4 g + t, column colp + e of this wave's partial product
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float* dst = &red[((wv * 16 + 4 * g + t) * 128) + n * 8];
      *reinterpret_cast<f32x4*>(dst) = f32x4{acc[0][t], acc[1][t], acc[2][t], acc[3][t]};
      *reinterpret_cast<f32x4*>(dst + 4) = f32x4{acc[4][t], acc[5][t], acc[6][t], acc[7][t]};
    }
  }
  __syncthreads();
  TR5(3);
  const int m = tid >> 5, c4 = (tid & 31) * 4;
  f32x4 tot = *reinterpret_cast<const f32x4*>(&red[m * 128 + c4]);
#pragma unroll
  for (int w = 1; w < DR_WAVES; ++w) tot += *reinterpret_cast<const f32x4*>(&red[(w * 16 + m) * 128 + c4]);
  const int col = col0 + c4;
  if (p.scales && mrow0 + m < p.M && c4 < cw && col < N) {
    const f16* sc = p.scales + (int64_t)bt * N + col;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (col + e < N) tot[e] *= (float)sc[e];
  }
  if (p.ep && mrow0 + m < p.M && c4 < cw && col < N) {
    const T* bias = reinterpret_cast<const T*>(p.bias);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (col + e < N) {
        float v = TypeTraits<T>::to_f32(TypeTraits<T>::from_f32(tot[e]));
        if (bias) v += TypeTraits<T>::to_f32(bias[(int64_t)bt * p.o_bs + (int64_t)(col + e) * p.o_ns]);
        tot[e] = apply_act(v, p.act);
      }
  }
  if (p.out_f32) {
    // (N is a multiple of 8 and col of 4: the four columns are all inside)
    if (mrow0 + m < p.M && c4 < cw && col < N)
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.out) + (int64_t)(mrow0 + m) * p.o_ms + (int64_t)bt * p.o_bs + col) = tot;
  } else if (mrow0 + m < p.M && c4 < cw && col < N) {
    T* o = reinterpret_cast<T*>(p.out) + (int64_t)(mrow0 + m) * p.o_ms + (int64_t)bt * p.o_bs;
    int ocol = col;
    if (p.per > 0) {                                     // (per is a multiple of 4: the four columns stay together)
      const uint32_t l = fd_div((uint32_t)col, p.perdiv);
      o = reinterpret_cast<T*>(p.out) + (int64_t)l * p.o_ls + (int64_t)(mrow0 + m) * p.o_ms + (int64_t)bt * p.per;
      ocol = col - (int)l * p.per;
    }
    if (p.o_ns == 1 && col + 3 < N && ((reinterpret_cast<uintptr_t>(o + ocol) & 7) == 0)) {
      typename TypeTraits<T>::vec4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = TypeTraits<T>::from_f32(tot[e]);
      *reinterpret_cast<typename TypeTraits<T>::vec4*>(o + ocol) = v;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < N) o[(int64_t)(ocol + e) * p.o_ns] = TypeTraits<T>::from_f32(tot[e]);
    }
  }
  if (!MULTI || !more) break;
  __syncthreads();                                       // red is free again
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < STEPS; ++s) av[s] = avn[s];
  products();                                            // (what does not depend on the tile - widening of codes, byte permutes - is
                                                         // moved in front of the loop by the compiler and done once)
  }  // tiles of 16 rows
  TR5(4);
}

// ---- warming the L2 for the second product ---------------------------------------------------------------------------------
// A launch between the two products that only adds slices (low rank, sliced Monarch) leaves the memory system idle.  Extra
// workgroups of that launch load the chunks of the second product's factor and drop the data: chunk of workgroup w2 of the next
// launch by a workgroup that runs on the same XCD (workgroup w of a launch runs on XCD w % 8 and each XCD has its own L2), up
// to a budget per workgroup that keeps an XCD's share within its L2.
struct RowsPrefetch {
  const char* W; int64_t w_bs_bytes;      // factor; bytes per batch entry
  uint32_t chunk_step, row_stride;        // bytes from chunk to chunk and from row to row of a chunk
  uint32_t piece16, last_piece16;         // 16-byte pieces per row of a chunk (of the last chunk of an entry)
  uint32_t nrows;                         // rows of a chunk
  uint32_t budget16;                      // at most this many pieces per workgroup
  FastDiv nch; uint32_t xcd_span;         // as in RowsParams of the launch that will read the chunks
  uint32_t nblocks2;                      // workgroups of that launch (0: nothing to fetch)
};

__device__ __forceinline__ void rows_prefetch(const RowsPrefetch& f, uint32_t first_block) {
  const uint32_t q = blockIdx.x, t = q - first_block;
  const uint32_t b2 = (t & ~7u) + (q & 7u);              // same XCD as workgroup b2 of the next launch
  if (b2 >= f.nblocks2) return;
  const uint32_t item = f.xcd_span ? (b2 & 7u) * f.xcd_span + (b2 >> 3) : b2;
  const uint32_t bt = fd_div(item, f.nch), ch = item - bt * f.nch.d;
  const uint32_t p16 = ch + 1 == f.nch.d ? f.last_piece16 : f.piece16;
  const char* base = f.W + (int64_t)bt * f.w_bs_bytes + (int64_t)ch * f.chunk_step;
  uint32_t units = f.nrows * p16;
  if (units > f.budget16) units = f.budget16;
  const uint32_t nt = blockDim.x;
  for (uint32_t u0 = threadIdx.x; u0 < units; u0 += 8 * nt) {
    u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t u = u0 + (uint32_t)k * nt;
      if (u < units) {
        const uint32_t row = u / p16, pc = u - row * p16;
        v[k] = *reinterpret_cast<const u32x4*>(base + (int64_t)row * f.row_stride + (int64_t)pc * 16);
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (u0 + (uint32_t)k * nt < units) asm volatile("" ::"v"(v[k]));
  }
}

// ---- the mix between the two products: z[i][m][r] = sum_j S(i, j, r) y[j][m][r], rank contiguous in S ------------------------
// One thread per VW (four or eight) ranks of one (i, m): 2 b loads of 2 VW bytes, all in flight at once, neighbouring threads on
// neighbouring ranks.  Y is re-read b times and S M times - from L2, both are a few hundred KiB.  fp32 sums in input-block order.
// (A load instruction costs a compute unit's address path the same whether a lane takes 8 or 16 bytes: eight ranks per thread in
// workgroups of 128 threads halve the instructions of every compute unit - the launcher takes them when there is enough work.)
template <typename T, int B, int VW>
__global__ __launch_bounds__(256) void rows_mix_kernel(const T* __restrict__ Y, const T* __restrict__ S, T* __restrict__ Z,
                                                        int M, int b, int R, int64_t s_si, int64_t s_sj, FastDiv r4div, FastDiv bdiv, uint32_t total,
                                                        RowsPrefetch pf, uint32_t nmix) {
  if (blockIdx.x >= nmix) { rows_prefetch(pf, nmix); return; }
  const uint32_t item = blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= total) return;
  const uint32_t t = fd_div(item, r4div), r4 = item - t * r4div.d;         // (r4: the thread's piece of VW ranks)
  const uint32_t m = fd_div(t, bdiv), i = t - m * bdiv.d;
  const T* sp = S + (int64_t)i * s_si + r4 * VW;
  const T* yp = Y + (int64_t)m * R + r4 * VW;
  const int64_t y_sj = (int64_t)M * R;
  float acc[VW];
#pragma unroll
  for (int e = 0; e < VW; ++e) acc[e] = 0.f;
  using V4 = typename std::conditional<VW == 8, typename TypeTraits<T>::vec8, typename TypeTraits<T>::vec4>::type;
  if constexpr (B > 0) {
    V4 sv[B], yv[B];
#pragma unroll
    for (int j = 0; j < B; ++j) { sv[j] = *reinterpret_cast<const V4*>(sp + j * s_sj); yv[j] = *reinterpret_cast<const V4*>(yp + j * y_sj); }
#pragma unroll
    for (int j = 0; j < B; ++j)
#pragma unroll
      for (int e = 0; e < VW; ++e) acc[e] += TypeTraits<T>::to_f32(sv[j][e]) * TypeTraits<T>::to_f32(yv[j][e]);
  } else {
    for (int j = 0; j < b; ++j) {
      const V4 sv = *reinterpret_cast<const V4*>(sp + j * s_sj), yv = *reinterpret_cast<const V4*>(yp + j * y_sj);
#pragma unroll
      for (int e = 0; e < VW; ++e) acc[e] += TypeTraits<T>::to_f32(sv[e]) * TypeTraits<T>::to_f32(yv[e]);
    }
  }
  V4 o;
#pragma unroll
  for (int e = 0; e < VW; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V4*>(Z + ((int64_t)i * M + m) * R + r4 * VW) = o;
}

// Low rank seen as BLAST with one output block and S = 1: z[m][r] = sum_j y[j][m][r] (the k-slices of x A).  The slices are
// fp32 partial sums, added in slice order and rounded to T once - the reduction is then accumulated in fp32 from end to end,
// as a single-pass product does (reference triton_funcs/low_rank_kernels.py:98-112, dense_kernels.py:80-98).
template <typename T>
__global__ __launch_bounds__(256) void rows_sum_kernel(const float* __restrict__ Y, T* __restrict__ Z, int b, int64_t MR4, RowsPrefetch pf, uint32_t nmix) {
  if (blockIdx.x >= nmix) { rows_prefetch(pf, nmix); return; }
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= MR4) return;
  using V4 = typename TypeTraits<T>::vec4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = 0; j0 < b; j0 += 8) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const f32x4*>(Y + ((int64_t)min(j0 + u, b - 1) * MR4 + item) * 4);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (j0 + u < b)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += v[u][e];
  }
  V4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V4*>(Z + item * 4) = o;
}

// Monarch with its input blocks cut into ks slices (so that the first product spreads over the chip): the slices are added and
// the permutation applied in one pass, z[l][m][r] = sum_s y[(r / per) ks + s][m][l per + r % per]; thread = four ranks.  The
// slices are fp32 partial sums (one rounding, after the sum).
template <typename T>
__global__ __launch_bounds__(256) void rows_perm_sum_kernel(const float* __restrict__ Y, T* __restrict__ Z, int ks, int M, int R, int per, int64_t items,
                                                            RowsPrefetch pf, uint32_t nmix) {
  if (blockIdx.x >= nmix) { rows_prefetch(pf, nmix); return; }
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (item >= items) return;
  using V4 = typename TypeTraits<T>::vec4;
  const int r4n = R >> 2;
  const int r = (int)(item % r4n) * 4;
  const int64_t lm = item / r4n;
  const int m = (int)(lm % M), l = (int)(lm / M);
  const int yj = r / per, yr = l * per + (r - yj * per);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < ks; ++s) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(Y + (((int64_t)(yj * ks + s) * M + m) * R + yr));
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += v[e];
  }
  V4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V4*>(Z + item * 4) = o;
}

// The same mix for S stored (r, i, j) - the input block contiguous (the layout of the bmm names and of the quantized
// entry points).  Neighbouring threads take neighbouring output blocks i, so that a wave reads whole (r, :, :) slices of S.
template <typename T>
__global__ __launch_bounds__(256) void rows_mix_rij_kernel(const T* __restrict__ Y, const T* __restrict__ S, T* __restrict__ Z,
                                                            int M, int R, FastDiv r4div, uint32_t total, RowsPrefetch pf, uint32_t nmix) {
  constexpr int B = 16;
  if (blockIdx.x >= nmix) { rows_prefetch(pf, nmix); return; }
  const uint32_t item = blockIdx.x * 256u + threadIdx.x;
  if (item >= total) return;
  const uint32_t i = item & (B - 1), t = item >> 4;
  const uint32_t m = fd_div(t, r4div), r4 = t - m * r4div.d;
  using V4 = typename TypeTraits<T>::vec4;
  using V8 = typename TypeTraits<T>::vec8;
  V8 sv[4][2];
  V4 yv[B];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const T* sp = S + ((int64_t)(r4 * 4 + e) * B + i) * B;
    sv[e][0] = *reinterpret_cast<const V8*>(sp); sv[e][1] = *reinterpret_cast<const V8*>(sp + 8);
  }
  const T* yp = Y + (int64_t)m * R + r4 * 4;
  const int64_t y_sj = (int64_t)M * R;
#pragma unroll
  for (int j = 0; j < B; ++j) yv[j] = *reinterpret_cast<const V4*>(yp + j * y_sj);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < B; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += TypeTraits<T>::to_f32(sv[e][j >> 3][j & 7]) * TypeTraits<T>::to_f32(yv[j][e]);
  V4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V4*>(Z + ((int64_t)i * M + m) * R + r4 * 4) = o;
}

namespace {

inline unsigned prefetch_blocks(const RowsPrefetch& pf) { return pf.nblocks2 ? (pf.nblocks2 + 7u) & ~7u : 0u; }

template <typename T>
int rows_mix_rij_t(const void* Y, const void* S, void* Z, int M, int R, const RowsPrefetch& pf, hipStream_t st) {
  const uint32_t total = (uint32_t)((int64_t)M * 16 * (R / 4));
  const uint32_t nmix = (uint32_t)cdiv(total, 256);
  hipLaunchKernelGGL((rows_mix_rij_kernel<T>), dim3(nmix + prefetch_blocks(pf)), dim3(256), 0, st, (const T*)Y, (const T*)S, (T*)Z, M, R,
                     fd_make((uint32_t)(R / 4)), total, pf, nmix);
  BLR_CHECK_LAUNCH("rows_mix_rij");
  return BLR_OK;
}

template <typename T>
int rows_mix_t(const void* Y, const void* S, void* Z, int M, int b, int R, int64_t s_si, int64_t s_sj, const RowsPrefetch& pf, hipStream_t st) {
  // eight ranks per thread once four would make more than two workgroups of 256 threads per compute unit (side by side at 64 rows:
  // 4096 -> 4096 20.4 -> 19.95 us, 4096 -> 22016 31.7 -> 30.5, 11008 -> 4096 30.1 -> 28.9; at 4 and 16 rows, where four ranks per
  // thread just fill the chip, the wider threads are 0.1 - 0.3 us slower)
  const bool wide = b == 16 && R % 8 == 0 && s_si % 8 == 0 && s_sj % 8 == 0 && aligned(Y, 16) && aligned(S, 16) && aligned(Z, 16) &&
                    (int64_t)M * b * (R / 4) >= 131072;
  const int vw = wide ? 8 : 4, nt = wide ? 128 : 256;
  const uint32_t total = (uint32_t)((int64_t)M * b * (R / vw));
  const uint32_t nmix = (uint32_t)cdiv(total, nt);
  const dim3 grid(nmix + prefetch_blocks(pf)), block(nt);
  const FastDiv r4div = fd_make((uint32_t)(R / vw)), bdiv = fd_make((uint32_t)b);
  if (wide) hipLaunchKernelGGL((rows_mix_kernel<T, 16, 8>), grid, block, 0, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, r4div, bdiv, total, pf, nmix);
  else if (b == 16) hipLaunchKernelGGL((rows_mix_kernel<T, 16, 4>), grid, block, 0, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, r4div, bdiv, total, pf, nmix);
  else hipLaunchKernelGGL((rows_mix_kernel<T, 0, 4>), grid, block, 0, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, r4div, bdiv, total, pf, nmix);
  BLR_CHECK_LAUNCH("rows_mix");
  return BLR_OK;
}

// Column pieces per chunk: the busiest compute unit's bytes bound the launch (35 GB/s each), short row pieces cost DRAM efficiency.
int plan_pieces(int batch, int K, int N, int wbits, int cus) {
  const int pieces = N / 8;
  int best = 16; double best_t = 1e30;
  for (int npc = 16; npc >= 2; --npc) {
    const int64_t chunks = (int64_t)batch * cdiv(pieces, npc);
    const double slab = (double)K * npc * wbits;      // bytes: 8 columns of wbits bits per piece and row
    double t = (double)cdiv(chunks, cus) * (0.5 + slab / 35e3);
    if (npc < 8) t += 0.05 * (8 - npc);
    // rows that start on cache-line boundaries: chunks whose row piece is not whole lines make neighbours fetch lines twice
    // (measured on 4 x (1024 x 5504): 176-byte pieces 24.4 us, 256-byte pieces 21.5 us for the whole call)
    if (((int64_t)N * wbits / 8) % 128 == 0 && (npc * wbits) % 128 != 0) t *= 1.45;
    if (t < best_t - 1e-9) { best_t = t; best = npc; }
  }
  return best;
}

template <typename T, int WB, bool NK, bool MULTI>
int rows_launch_m(RowsParams& p, int batch, hipStream_t st) {
  const int steps = p.kw / 32;
  const dim3 grid((unsigned)(batch * p.nch.d)), block(DR_NT);
  switch (steps) {
    case 1: hipLaunchKernelGGL((rows_product_kernel<T, 1, WB, NK, MULTI>), grid, block, 0, st, p); break;
    case 2: hipLaunchKernelGGL((rows_product_kernel<T, 2, WB, NK, MULTI>), grid, block, 0, st, p); break;
    case 3: hipLaunchKernelGGL((rows_product_kernel<T, 3, WB, NK, MULTI>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((rows_product_kernel<T, 4, WB, NK, MULTI>), grid, block, 0, st, p); break;
  }
  BLR_CHECK_LAUNCH("rows_product");
  return BLR_OK;
}
template <typename T, int WB, bool NK = false>
int rows_launch_t(RowsParams& p, int batch, hipStream_t st) {
  return p.mtiles > 1 ? rows_launch_m<T, WB, NK, true>(p, batch, st) : rows_launch_m<T, WB, NK, false>(p, batch, st);
}

// Plans one batch of skinny products (chunk width, rounds, item order); returns 1 when the operands do not fit the kernel.
int rows_plan(RowsParams& p, int batch, int dtype, int wbits, bool nk) {
  if (nk && wbits != 16) return 1;
  if (p.K % 8 || p.N % 8 || p.N > 65536 || p.K > 4 * DR_WAVES * DR_MAX_STEPS * 32) return 1;
  if (!aligned(p.A, 16) || !aligned(p.W, 16) || p.lda % 8 || p.a_bs % 8 || p.w_bs % 32) return 1;
  if ((int64_t)p.K * p.N * 2 >= (int64_t)DR_OOB) return 1;
  if (wbits != 16 && dtype != BLR_F16 && dtype != BLR_BF16) return 1;
  p.rounds = (int)cdiv(p.K, DR_WAVES * DR_MAX_STEPS * 32);
  p.mtiles = (int)cdiv(p.M, 16);
  if (p.mtiles > 1 && p.rounds > 1) return 1;          // more rows than one tile only with the whole factor slice in registers
  p.kw = (int)cdiv(cdiv(p.K, DR_WAVES * p.rounds), 32) * 32;
  const int cus = device_cus() > 0 ? device_cus() : 256;
  if (nk) {
    // column groups of 16 per chunk (at most 8): as many as keep the busiest compute unit's bytes lowest
    int best = 8; double best_t = 1e30;
    for (int cg = 8; cg >= 1; --cg) {
      const double t = (double)cdiv((int64_t)batch * cdiv(p.N, 16 * cg), cus) * (0.5 + (double)p.K * cg * 32.0 / 35e3);
      if (t < best_t - 1e-9) { best_t = t; best = cg; }
    }
    p.npc = best;
    p.nch = fd_make((uint32_t)cdiv(p.N, 16 * p.npc));
  } else {
    p.npc = plan_pieces(batch, p.K, p.N, wbits, cus);
    p.nch = fd_make((uint32_t)cdiv(p.N / 8, p.npc));
  }
  if ((int64_t)batch * p.nch.d >= 65536) return 1;
  p.xcd_span = ((batch * p.nch.d) % 8 == 0) ? (uint32_t)(batch * p.nch.d / 8) : 0u;
  return BLR_OK;
}

int rows_launch(RowsParams p, int batch, int dtype, int wbits, bool nk, hipStream_t st) {
  if (nk) return dtype == BLR_F16 ? rows_launch_t<f16, 16, true>(p, batch, st) : rows_launch_t<bf16, 16, true>(p, batch, st);
  if (wbits == 16) return dtype == BLR_F16 ? rows_launch_t<f16, 16>(p, batch, st) : rows_launch_t<bf16, 16>(p, batch, st);
  if (wbits == 8) return dtype == BLR_F16 ? rows_launch_t<f16, 8>(p, batch, st) : rows_launch_t<bf16, 8>(p, batch, st);
  return dtype == BLR_F16 ? rows_launch_t<f16, 4>(p, batch, st) : rows_launch_t<bf16, 4>(p, batch, st);
}

// What the launch before a planned product can fetch ahead for it; nblocks2 = 0 when the chunks are not whole 16-byte pieces
// or the factor is too small to matter.
RowsPrefetch rows_prefetch_plan(const RowsParams& p, int batch, int wbits, bool nk) {
  RowsPrefetch f = {};
  static const int enabled = 1;
  if (!enabled) return f;
  const int64_t w_bytes = (int64_t)batch * p.K * p.N * wbits / 8;
  if (w_bytes < (1 << 20)) return f;
  f.W = reinterpret_cast<const char*>(p.W); f.w_bs_bytes = p.w_bs * wbits / 8;
  if (nk) {                                              // chunk = 16 npc whole rows of K elements: one contiguous run
    const int cw = p.npc * 16;
    f.chunk_step = (uint32_t)((int64_t)cw * p.K * 2); f.row_stride = 0; f.nrows = 1;
    f.piece16 = f.chunk_step / 16;
    f.last_piece16 = (uint32_t)((int64_t)(p.N - (int)(p.nch.d - 1) * cw) * p.K * 2 / 16);
  } else {                                               // chunk = K rows of 8 npc columns
    const int cw = p.npc * 8;
    const int64_t piece = (int64_t)cw * wbits / 8, row = (int64_t)p.N * wbits / 8;
    if (piece % 16 || row % 16 || f.w_bs_bytes % 16) return f;
    f.chunk_step = (uint32_t)piece; f.row_stride = (uint32_t)row; f.nrows = (uint32_t)p.K;
    f.piece16 = (uint32_t)(piece / 16);
    f.last_piece16 = (uint32_t)((row - (int64_t)(p.nch.d - 1) * piece) / 16);
  }
  f.nch = p.nch; f.xcd_span = p.xcd_span;
  f.nblocks2 = (uint32_t)batch * p.nch.d;
  // per workgroup: what a compute unit draws during the launch (about 35 GB/s for 2 - 3 us), and an XCD's share within 3 MB of its L2
  int64_t budget = (int64_t)96 * 1024;
  const int64_t per_xcd = (int64_t)3 << 20;
  if (budget * ((f.nblocks2 + 7) / 8) > per_xcd) budget = per_xcd / ((f.nblocks2 + 7) / 8);
  f.budget16 = (uint32_t)(budget / 16);
  if (f.budget16 == 0) f.nblocks2 = 0;
  return f;
}

}  // namespace

int decode_rows_launch(const StreamBlastArgs& a, void* region, size_t region_bytes, hipStream_t st) {
  const int enabled = option_value(OPT_DECODE_ROWS, 1);
  if (!enabled) return 1;
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int b = a.b, M = a.M, R = a.r, P = a.in_f / a.b, Q = a.out_f / bo;
  const bool u_nk = a.u_layout == BLR_U_QR;
  const bool monarch = a.perm_per > 0;                  // the mix is a permutation, folded into the store of the first product
  const bool lowrank = !monarch && !a.S && bo == 1;     // one output block, S = 1: the mix is the sum over the input slices
  if (M < 1 || M > DR_MAX_M || (!monarch && !lowrank && !a.S) || (bo != b && !lowrank) || (u_nk && a.wbits != 16)) return 1;
  if (lowrank && a.wbits != 16) return 1;
  if (monarch && (a.wbits != 16 || a.perm_per % 4 || R % a.perm_per || R / a.perm_per != b || a.perm_per >= 65536)) return 1;
  if (a.wbits != 16 && (!a.u_scales || !a.v_scales)) return 1;
  if (a.dtype != BLR_F16 && a.dtype != BLR_BF16) return 1;
  // Monarch with input blocks deeper than one round of the product kernel (1024 rows): few, long chunks would leave most of the
  // chip idle (4 blocks x 8 chunks at 11008 -> 4096), so each block is cut into ks equal slices of whole 16-byte pieces and the
  // slices are added where the permutation is applied (24.3 -> 18.4 us at 16 rows there)
  int mks = 1;
  if (monarch && P > 1024) {                            // (cutting shallower blocks too measured 0.3 - 0.4 us slower)
    for (int ks = (P + 1023) / 1024; ks <= 8; ++ks)
      if (P % ks == 0 && (P / ks) % 8 == 0) { mks = ks; break; }
  }
  const bool y_f32 = lowrank || mks > 1;                // y holds slices of one reduction: fp32 partial sums, rounded once after their sum
  const size_t ybytes = align_up((size_t)b * mks * M * R * (y_f32 ? 4 : 2), 256), zbytes = align_up((size_t)bo * M * R * 2, 256);
  if (ybytes + zbytes > region_bytes) return 1;
  void* Y = region;
  void* Z = reinterpret_cast<char*>(region) + ybytes;
  const int64_t x_elems = (int64_t)(M - 1) * a.ldx + a.in_f;
  if (x_elems * 2 >= (int64_t)DR_OOB) return 1;

  RowsParams s1 = {};
  s1.A = a.x; s1.lda = a.ldx; s1.a_bs = P; s1.a_bytes = (uint32_t)(x_elems * 2);
  s1.W = a.V; s1.w_bs = (int64_t)P * R;
  s1.out = Y; s1.o_ms = R; s1.o_bs = (int64_t)M * R; s1.o_ns = 1;
  s1.M = M; s1.K = P; s1.N = R; s1.scales = a.wbits != 16 ? (const f16*)a.v_scales : nullptr;
  if (monarch && mks == 1) { s1.out = Z; s1.o_bs = 0; s1.per = a.perm_per; s1.o_ls = (int64_t)M * R; s1.perdiv = fd_make((uint32_t)a.perm_per); }
  if (mks > 1) { s1.a_bs = P / mks; s1.w_bs = (int64_t)(P / mks) * R; s1.K = P / mks; }
  s1.out_f32 = y_f32 ? 1 : 0;
  RowsParams s2 = {};
  s2.A = Z; s2.lda = R; s2.a_bs = (int64_t)M * R; s2.a_bytes = (uint32_t)((size_t)bo * M * R * 2);
  s2.W = a.U; s2.w_bs = (int64_t)R * Q;
  s2.out = a.out; s2.o_ms = a.ldo;
  s2.o_bs = a.out_ns ? a.out_bs : Q; s2.o_ns = a.out_ns ? a.out_ns : 1;
  s2.M = M; s2.K = R; s2.N = Q; s2.trace_base = 512; s2.scales = a.wbits != 16 ? (const f16*)a.u_scales : nullptr;
  // both products must fit before the first launch
  if (P % 8 || R % 8 || Q % 8 || P > 4096 || R > 4096 || !aligned(a.x, 16) || !aligned(a.V, 16) || !aligned(a.U, 16) || a.ldx % 8) return 1;

  const void* ep_bias = nullptr; int ep_act = 0;
  if (epilogue_pending(&ep_bias, &ep_act)) { s2.ep = 1; s2.bias = ep_bias; s2.act = ep_act; }
  int rc = rows_plan(s1, b * mks, a.dtype, a.wbits, false);
  if (rc) return rc;
  rc = rows_plan(s2, bo, a.dtype, a.wbits, u_nk);
  if (rc) return rc;
  // Fetching ahead pays where the launch in between is trivial (the sum of slices of low rank and of sliced Monarch) and the
  // factor small: 11008 -> 4096 at 16 rows, low rank 18.8 -> 17.6 us, Monarch 18.6 -> 17.6 us.  Next to the BLAST mix, which is
  // itself waiting on memory, it costs more than it gives (4096 -> 22016: 20.0 -> 21.9 us; 11008 -> 4096: 17.8 -> 18.3 us).
  const bool ahead = (lowrank || (monarch && mks > 1)) && (int64_t)bo * R * Q * a.wbits / 8 <= (int64_t)12 << 20;
  const RowsPrefetch pf = ahead ? rows_prefetch_plan(s2, bo, a.wbits, u_nk) : RowsPrefetch{};
  rc = rows_launch(s1, b * mks, a.dtype, a.wbits, false, st);
  if (rc) return rc;
  int64_t si, sj, sr;
  if (a.s_layout == BLR_S_JIR) { sj = (int64_t)b * R; si = R; sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { sr = (int64_t)b * b; si = b; sj = 1; }
  else { si = (int64_t)b * R; sj = R; sr = 1; }
  if (monarch && mks > 1) {
    const int64_t items = (int64_t)bo * M * R / 4;
    const uint32_t nmix = (uint32_t)cdiv(items, 256);
    if (a.dtype == BLR_F16) hipLaunchKernelGGL(rows_perm_sum_kernel<f16>, dim3(nmix + prefetch_blocks(pf)), dim3(256), 0, st, (const float*)Y, (f16*)Z, mks, M, R, a.perm_per, items, pf, nmix);
    else hipLaunchKernelGGL(rows_perm_sum_kernel<bf16>, dim3(nmix + prefetch_blocks(pf)), dim3(256), 0, st, (const float*)Y, (bf16*)Z, mks, M, R, a.perm_per, items, pf, nmix);
    BLR_CHECK_LAUNCH("rows_perm_sum");
  } else if (monarch)
    rc = BLR_OK;
  else if (lowrank) {
    const int64_t mr4 = (int64_t)M * R / 4;
    const uint32_t nmix = (uint32_t)cdiv(mr4, 256);
    if (a.dtype == BLR_F16) hipLaunchKernelGGL(rows_sum_kernel<f16>, dim3(nmix + prefetch_blocks(pf)), dim3(256), 0, st, (const float*)Y, (f16*)Z, b, mr4, pf, nmix);
    else hipLaunchKernelGGL(rows_sum_kernel<bf16>, dim3(nmix + prefetch_blocks(pf)), dim3(256), 0, st, (const float*)Y, (bf16*)Z, b, mr4, pf, nmix);
    BLR_CHECK_LAUNCH("rows_sum");
  } else if (sr == 1 && si % 4 == 0 && sj % 4 == 0 && R % 4 == 0 && aligned(a.S, 8) && (int64_t)M * b * (R / 4) * (R / 4) < ((int64_t)1 << 32) && b < 65536)   // the multiply-high division is exact below 2^32 / divisor
    rc = a.dtype == BLR_F16 ? rows_mix_t<f16>(Y, a.S, Z, M, b, R, si, sj, pf, st) : rows_mix_t<bf16>(Y, a.S, Z, M, b, R, si, sj, pf, st);
  else if (a.s_layout == BLR_S_RIJ && b == 16 && R % 4 == 0 && aligned(a.S, 16) && (int64_t)M * (R / 4) * (R / 4) < ((int64_t)1 << 32))
    rc = a.dtype == BLR_F16 ? rows_mix_rij_t<f16>(Y, a.S, Z, M, R, pf, st) : rows_mix_rij_t<bf16>(Y, a.S, Z, M, R, pf, st);
  else
    rc = blast_mix_launch(Y, a.S, Z, M, b, R, si, sj, sr, a.dtype, st, 0);
  if (rc) return rc;
  rc = rows_launch(s2, bo, a.dtype, a.wbits, u_nk, st);
  if (rc == BLR_OK && s2.ep) epilogue_taken();
  return rc == 1 ? BLR_ERR_UNSUPPORTED : rc;
}

// ---- dense at 17..128 rows ----------------------------------------------------------------------------------------------
namespace {
int dense_slices(int in_f) {
  for (int c = 1; c <= 16; ++c)
    if (in_f % c == 0 && (in_f / c) % 8 == 0 && in_f / c <= 1024) return c;
  return 0;
}
}  // namespace

// Measured against the 256-row tiles (us at 17 / 64 / 128 rows): 4096 -> 4096 13 / 17 / 23 against 47 / 49 / 56, 11008 -> 4096
// 26 / 33 / 44 against 116 / 124 / 144, 4096 -> 22016 46 / 58 / 77 against 54 / 56 / 63 - a wide output has enough tiles of its own
// and pays for the slices' partial products, so it comes here only up to 48 rows.
static bool dense_rows_wanted(int M, int out_f) { return M > 16 && M <= DR_MAX_M && (out_f <= 8192 || M <= 48); }

size_t dense_rows_bytes(int M, int in_f, int out_f, int dtype) {
  const int bi = dense_slices(in_f);
  if (!dense_rows_wanted(M, out_f) || (dtype != BLR_F16 && dtype != BLR_BF16) || !bi || out_f % 8) return 0;
  return bi > 1 ? align_up((size_t)bi * M * out_f * 4, 256) : 0;    // fp32 partial sums of the slices
}

int dense_rows_launch(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo, int M, int in_f, int out_f, int dtype,
                      void* ws, size_t ws_bytes, hipStream_t st) {
  const int enabled = option_value(OPT_DENSE_ROWS, 1);
  const int bi = dense_slices(in_f);
  if (!enabled || !dense_rows_wanted(M, out_f) || (dtype != BLR_F16 && dtype != BLR_BF16) || !bi || out_f % 8) return 1;
  if (bi > 1 && (ldo != out_f || !ws || ws_bytes < dense_rows_bytes(M, in_f, out_f, dtype) || !aligned(out, 8))) return 1;
  const int64_t x_elems = (int64_t)(M - 1) * ldx + in_f;
  if (x_elems * 2 >= (int64_t)DR_OOB || ldx % 8 || !aligned(x, 16) || !aligned(W, 16)) return 1;
  RowsParams s = {};
  s.A = x; s.lda = ldx; s.a_bs = in_f / bi; s.a_bytes = (uint32_t)(x_elems * 2);
  s.W = W; s.w_bs = (int64_t)(in_f / bi) * out_f;
  s.out = bi > 1 ? ws : out; s.o_ms = bi > 1 ? out_f : ldo; s.o_bs = (int64_t)M * out_f; s.o_ns = 1;
  s.M = M; s.K = in_f / bi; s.N = out_f; s.out_f32 = bi > 1 ? 1 : 0;
  const void* ep_bias = nullptr; int ep_act = 0;
  if (bi == 1 && epilogue_pending(&ep_bias, &ep_act)) { s.ep = 1; s.bias = ep_bias; s.act = ep_act; }
  int rc = rows_plan(s, bi, dtype, 16, false);
  if (rc) return rc;
  rc = rows_launch(s, bi, dtype, 16, false, st);
  if (rc) return rc == 1 ? BLR_ERR_UNSUPPORTED : rc;
  if (bi == 1) { if (s.ep) epilogue_taken(); return BLR_OK; }
  const int64_t mn4 = (int64_t)M * out_f / 4;
  const uint32_t nsum = (uint32_t)cdiv(mn4, 256);
  const RowsPrefetch none = {};
  if (dtype == BLR_F16) hipLaunchKernelGGL(rows_sum_kernel<f16>, dim3(nsum), dim3(256), 0, st, (const float*)ws, (f16*)out, bi, mn4, none, nsum);
  else hipLaunchKernelGGL(rows_sum_kernel<bf16>, dim3(nsum), dim3(256), 0, st, (const float*)ws, (bf16*)out, bi, mn4, none, nsum);
  BLR_CHECK_LAUNCH("rows_sum");
  return BLR_OK;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace5(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace5), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

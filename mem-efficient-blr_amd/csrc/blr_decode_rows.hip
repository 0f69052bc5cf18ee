// BLAST at 5 to 16 token rows as three launches: y = x V on the matrix cores, the rank-space mix, out = z U on the matrix cores.
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
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
constexpr int DR_NT = 512;
constexpr int DR_WAVES = 8;
constexpr int DR_MAX_STEPS = 4;           // 32-row steps of a wave: 8 loads per lane each
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
  const void* W; int64_t w_bs;            // W[bt * w_bs + k * N + n]
  void* out; int64_t o_ms, o_bs, o_ns;    // out[m * o_ms + bt * o_bs + n * o_ns]
  int M, K, N;
  int kw;                                 // rows of a wave's share (a multiple of 32)
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

template <typename T, int STEPS>
__global__ __launch_bounds__(DR_NT) void rows_product_kernel(RowsParams p) {
  __shared__ __attribute__((aligned(16))) float red[DR_WAVES * 16 * 128];
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
  TR5(0);
  // workgroup w runs on XCD w % 8: neighbouring chunks (which share cache lines when a chunk's row piece is not a whole
  // number of lines) go to one XCD, i.e. one L2
  const uint32_t item = p.xcd_span ? (blockIdx.x & 7u) * p.xcd_span + (blockIdx.x >> 3) : blockIdx.x;
  const uint32_t bt = fd_div(item, p.nch), ch = item - bt * p.nch.d;
  const int N = p.N, K = p.K;
  const int col0 = (int)ch * p.npc * 8;                  // first column of the chunk
  const int colp = col0 + n * 8;                         // first column of this lane's pieces
  const bool live = n < p.npc && colp < N;
  const __amdgpu_buffer_rsrc_t abuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.A), 0, p.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wb = wbuf(reinterpret_cast<const char*>(p.W) + (int64_t)bt * p.w_bs * 2, (uint32_t)((int64_t)K * N * 2));
  const int kb = wv * p.kw + 8 * g;                      // first of this lane's eight k of step 0

  // activations: row n of A, the lane's eight k of every step (16 bytes each); weights: eight rows per step, the lane's
  // 16-byte piece of each.  Lanes without a row / without a column piece issue nothing (their registers stay undefined:
  // they only reach rows and columns of the product that are never stored), so a narrow chunk costs the load path
  // only what its live lanes fetch.
  u32x4 av[STEPS];
  u32x4 wr[STEPS][8];
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
  if (live) {
    const uint32_t wbase = (uint32_t)(kb * N + colp) * 2u;
    const uint32_t rowb = (uint32_t)N * 2u;
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < 8; ++t) wr[s][t] = ldw16(wb, wbase + (uint32_t)(32 * s + t) * rowb, 0);
  }

  TR5(1);
  f32x4 acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
      u32x4 bv;
#pragma unroll
      for (int h = 0; h < 4; ++h) bv[h] = __builtin_amdgcn_perm(wr[s][2 * h + 1][e >> 1], wr[s][2 * h][e >> 1], sel);
      acc[e] = RowsMfma<T>::run(av[s], bv, acc[e]);
    }
  }
  TR5(2);
  // acc[e][t] is row 4 g + t, column colp + e of this wave's partial product
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float* dst = &red[((wv * 16 + 4 * g + t) * 128) + n * 8];
    *reinterpret_cast<f32x4*>(dst) = f32x4{acc[0][t], acc[1][t], acc[2][t], acc[3][t]};
    *reinterpret_cast<f32x4*>(dst + 4) = f32x4{acc[4][t], acc[5][t], acc[6][t], acc[7][t]};
  }
  __syncthreads();
  TR5(3);
  const int m = tid >> 5, c4 = (tid & 31) * 4;
  f32x4 tot = *reinterpret_cast<const f32x4*>(&red[m * 128 + c4]);
#pragma unroll
  for (int w = 1; w < DR_WAVES; ++w) tot += *reinterpret_cast<const f32x4*>(&red[(w * 16 + m) * 128 + c4]);
  const int col = col0 + c4;
  if (m < p.M && c4 < p.npc * 8 && col < N) {
    T* o = reinterpret_cast<T*>(p.out) + (int64_t)m * p.o_ms + (int64_t)bt * p.o_bs;
    if (p.o_ns == 1 && col + 3 < N && ((reinterpret_cast<uintptr_t>(o + col) & 7) == 0)) {
      typename TypeTraits<T>::vec4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = TypeTraits<T>::from_f32(tot[e]);
      *reinterpret_cast<typename TypeTraits<T>::vec4*>(o + col) = v;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < N) o[(int64_t)(col + e) * p.o_ns] = TypeTraits<T>::from_f32(tot[e]);
    }
  }
  TR5(4);
}

// ---- the mix between the two products: z[i][m][r] = sum_j S(i, j, r) y[j][m][r], rank contiguous in S ------------------------
// One thread per four ranks of one (i, m): 2 b eight-byte loads, all in flight at once, neighbouring threads on neighbouring
// ranks.  Y is re-read b times and S M times - from L2, both are a few hundred KiB.  fp32 sums in input-block order.
template <typename T, int B>
__global__ __launch_bounds__(256) void rows_mix_kernel(const T* __restrict__ Y, const T* __restrict__ S, T* __restrict__ Z,
                                                        int M, int b, int R, int64_t s_si, int64_t s_sj, FastDiv r4div, FastDiv bdiv, uint32_t total) {
  const uint32_t item = blockIdx.x * 256u + threadIdx.x;
  if (item >= total) return;
  const uint32_t t = fd_div(item, r4div), r4 = item - t * r4div.d;
  const uint32_t m = fd_div(t, bdiv), i = t - m * bdiv.d;
  const T* sp = S + (int64_t)i * s_si + r4 * 4;
  const T* yp = Y + (int64_t)m * R + r4 * 4;
  const int64_t y_sj = (int64_t)M * R;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  using V4 = typename TypeTraits<T>::vec4;
  if constexpr (B > 0) {
    V4 sv[B], yv[B];
#pragma unroll
    for (int j = 0; j < B; ++j) { sv[j] = *reinterpret_cast<const V4*>(sp + j * s_sj); yv[j] = *reinterpret_cast<const V4*>(yp + j * y_sj); }
#pragma unroll
    for (int j = 0; j < B; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += TypeTraits<T>::to_f32(sv[j][e]) * TypeTraits<T>::to_f32(yv[j][e]);
  } else {
    for (int j = 0; j < b; ++j) {
      const V4 sv = *reinterpret_cast<const V4*>(sp + j * s_sj), yv = *reinterpret_cast<const V4*>(yp + j * y_sj);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += TypeTraits<T>::to_f32(sv[e]) * TypeTraits<T>::to_f32(yv[e]);
    }
  }
  V4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V4*>(Z + ((int64_t)i * M + m) * R + r4 * 4) = o;
}

namespace {

template <typename T>
int rows_mix_t(const void* Y, const void* S, void* Z, int M, int b, int R, int64_t s_si, int64_t s_sj, hipStream_t st) {
  const uint32_t total = (uint32_t)((int64_t)M * b * (R / 4));
  const dim3 grid((unsigned)cdiv(total, 256)), block(256);
  const FastDiv r4div = fd_make((uint32_t)(R / 4)), bdiv = fd_make((uint32_t)b);
  if (b == 16) hipLaunchKernelGGL((rows_mix_kernel<T, 16>), grid, block, 0, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, r4div, bdiv, total);
  else hipLaunchKernelGGL((rows_mix_kernel<T, 0>), grid, block, 0, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, r4div, bdiv, total);
  BLR_CHECK_LAUNCH("rows_mix");
  return BLR_OK;
}

// Column pieces per chunk: the busiest compute unit's bytes bound the launch (35 GB/s each), short row pieces cost DRAM efficiency.
int plan_pieces(int batch, int K, int N, int cus) {
  const int pieces = N / 8;
  int best = 16; double best_t = 1e30;
  for (int npc = 16; npc >= 2; --npc) {
    const int64_t chunks = (int64_t)batch * cdiv(pieces, npc);
    const double slab = (double)K * npc * 16.0;
    double t = (double)cdiv(chunks, cus) * (0.5 + slab / 35e3);
    if (npc < 8) t += 0.05 * (8 - npc);
    if (t < best_t - 1e-9) { best_t = t; best = npc; }
  }
  return best;
}

template <typename T>
int rows_launch_t(RowsParams& p, int batch, hipStream_t st) {
  const int steps = p.kw / 32;
  const dim3 grid((unsigned)(batch * p.nch.d)), block(DR_NT);
  switch (steps) {
    case 1: hipLaunchKernelGGL((rows_product_kernel<T, 1>), grid, block, 0, st, p); break;
    case 2: hipLaunchKernelGGL((rows_product_kernel<T, 2>), grid, block, 0, st, p); break;
    case 3: hipLaunchKernelGGL((rows_product_kernel<T, 3>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((rows_product_kernel<T, 4>), grid, block, 0, st, p); break;
  }
  BLR_CHECK_LAUNCH("rows_product");
  return BLR_OK;
}

// One batch of skinny products; returns 1 when the operands do not fit the kernel.
int rows_product(RowsParams p, int batch, int dtype, hipStream_t st) {
  if (p.K % 8 || p.N % 8 || p.N > 65536 || p.K > DR_WAVES * DR_MAX_STEPS * 32) return 1;
  if (!aligned(p.A, 16) || !aligned(p.W, 16) || p.lda % 8 || p.a_bs % 8 || p.w_bs % 8) return 1;
  if ((int64_t)p.K * p.N * 2 >= (int64_t)DR_OOB) return 1;
  p.kw = (int)cdiv(cdiv(p.K, DR_WAVES), 32) * 32;
  const int cus = device_cus() > 0 ? device_cus() : 256;
  static const int e_npc = env_i("BLR_DR_NPC", 0);
  p.npc = e_npc > 0 && e_npc <= 16 ? e_npc : plan_pieces(batch, p.K, p.N, cus);
  p.nch = fd_make((uint32_t)cdiv(p.N / 8, p.npc));
  if ((int64_t)batch * p.nch.d >= 65536) return 1;
  static const int e_xcd = env_i("BLR_DR_XCD", 1);
  p.xcd_span = (e_xcd && (batch * p.nch.d) % 8 == 0) ? (uint32_t)(batch * p.nch.d / 8) : 0u;
  return dtype == BLR_F16 ? rows_launch_t<f16>(p, batch, st) : rows_launch_t<bf16>(p, batch, st);
}

}  // namespace

int decode_rows_launch(const StreamBlastArgs& a, void* region, size_t region_bytes, hipStream_t st) {
  static const int enabled = env_i("BLR_DECODE_ROWS", 1);
  if (!enabled) return 1;
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int b = a.b, M = a.M, R = a.r, P = a.in_f / a.b, Q = a.out_f / bo;
  if (M < 1 || M > 16 || a.wbits != 16 || a.u_layout != BLR_U_RQ || a.perm_per > 0 || !a.S || bo != b) return 1;
  if (a.dtype != BLR_F16 && a.dtype != BLR_BF16) return 1;
  const size_t ybytes = align_up((size_t)b * M * R * 2, 256);
  if (2 * ybytes > region_bytes) return 1;
  void* Y = region;
  void* Z = reinterpret_cast<char*>(region) + ybytes;
  const int64_t x_elems = (int64_t)(M - 1) * a.ldx + a.in_f;
  if (x_elems * 2 >= (int64_t)DR_OOB) return 1;

  RowsParams s1 = {};
  s1.A = a.x; s1.lda = a.ldx; s1.a_bs = P; s1.a_bytes = (uint32_t)(x_elems * 2);
  s1.W = a.V; s1.w_bs = (int64_t)P * R;
  s1.out = Y; s1.o_ms = R; s1.o_bs = (int64_t)M * R; s1.o_ns = 1;
  s1.M = M; s1.K = P; s1.N = R;
  RowsParams s2 = {};
  s2.A = Z; s2.lda = R; s2.a_bs = (int64_t)M * R; s2.a_bytes = (uint32_t)((size_t)b * M * R * 2);
  s2.W = a.U; s2.w_bs = (int64_t)R * Q;
  s2.out = a.out; s2.o_ms = a.ldo;
  s2.o_bs = a.out_ns ? a.out_bs : Q; s2.o_ns = a.out_ns ? a.out_ns : 1;
  s2.M = M; s2.K = R; s2.N = Q; s2.trace_base = 512;
  // both products must fit before the first launch
  if (P % 8 || R % 8 || Q % 8 || P > 1024 || R > 1024 || !aligned(a.x, 16) || !aligned(a.V, 16) || !aligned(a.U, 16) || a.ldx % 8) return 1;

  int rc = rows_product(s1, b, a.dtype, st);
  if (rc) return rc;
  int64_t si, sj, sr;
  if (a.s_layout == BLR_S_JIR) { sj = (int64_t)b * R; si = R; sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { sr = (int64_t)b * b; si = b; sj = 1; }
  else { si = (int64_t)b * R; sj = R; sr = 1; }
  if (sr == 1 && si % 4 == 0 && sj % 4 == 0 && R % 4 == 0 && aligned(a.S, 8) && (int64_t)M * b * (R / 4) * (R / 4) < ((int64_t)1 << 32) && b < 65536)   // the multiply-high division is exact below 2^32 / divisor
    rc = a.dtype == BLR_F16 ? rows_mix_t<f16>(Y, a.S, Z, M, b, R, si, sj, st) : rows_mix_t<bf16>(Y, a.S, Z, M, b, R, si, sj, st);
  else
    rc = blast_mix_launch(Y, a.S, Z, M, b, R, si, sj, sr, a.dtype, st, 0);
  if (rc) return rc;
  rc = rows_product(s2, b, a.dtype, st);
  return rc == 1 ? BLR_ERR_UNSUPPORTED : rc;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace5(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace5), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

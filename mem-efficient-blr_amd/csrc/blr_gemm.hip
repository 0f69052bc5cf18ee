// Tiled batched GEMM for the prefill-sized (M > 16) shapes and for the fp32 verification
// variants, plus the BLAST rank-space mix used by the unfused (TILED) algorithm.
//
// f16 / bf16: 256-thread workgroups (4 waves as 2x2), v_mfma_f32_32x32x16 tiles, operands
// staged through LDS as [row][64 + 8] two-byte elements (the 16-byte pad makes the 128-bit
// fragment reads bank-conflict free).  Activations and (b,q,r)-style weights are K-contiguous
// and copied straight in; (k, n)-ordered weights (n contiguous - the layout most of the
// reference's kernel names use) are transposed in registers on their way into LDS.
// fp32: plain FMA tiles, used only by the *_fp32 verification names.
#include <cstdlib>
#include <mutex>
#include <set>
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_ring_dev.h"

namespace blr {

constexpr int BK = 64;          // k extent of an LDS tile
constexpr int LDS_LD = BK + 8;  // row stride in elements

template <typename T, int BM, int BN>
struct GemmSmem {
  T a[BM][LDS_LD];
  T b[BN][LDS_LD];
};

// ---- global -> register staging ------------------------------------------------------------
// Both stagers keep per-thread base pointers computed once (rows / columns outside the problem
// are clamped to the last valid one - their results are never stored), so that a full k tile is
// fetched with unconditional 16-byte loads at a uniform offset.  Only the last, partial k tile
// and operands that are not 16-byte friendly take the guarded element-wise path.
//
// K-contiguous operand: tile of ROWS rows x 64 k.  Thread t owns vectors v = t + i*256,
// row = v / 8, k-vector = v % 8 (8 lanes cover one 128-byte row segment).
template <typename T, int ROWS>
struct KcStage {
  static constexpr int NV = ROWS * 8 / 256;
  using V8 = typename TypeTraits<T>::vec8;
  struct Vals { V8 v[NV]; };
  const T* p[NV];

  __device__ __forceinline__ void init(const T* base, int64_t ld, int row0, int nrows, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int vi = tid + i * 256;
      int row = vi >> 3, kv = (vi & 7) * 8;
      p[i] = base + (int64_t)min(row0 + row, nrows - 1) * ld + kv;
    }
  }
  // full tile, 16-byte friendly operand: no conditions, so the number of loads in flight is known statically
  __device__ __forceinline__ void load_vec(Vals& r, int k0) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) r.v[i] = ldg16<V8>(p[i] + k0);
  }
  __device__ __forceinline__ void load(Vals& r, int k0, int K, bool vec_ok, int tid) const {
    if (vec_ok && k0 + BK <= K) {
#pragma unroll
      for (int i = 0; i < NV; ++i) r.v[i] = ldg16<V8>(p[i] + k0);
      return;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int kv = ((tid + i * 256) & 7) * 8;
      int gk = k0 + kv;
      V8 val;
#pragma unroll
      for (int e = 0; e < 8; ++e) val[e] = (gk + e < K) ? p[i][k0 + e] : (T)0.0f;
      r.v[i] = val;
    }
  }
  __device__ __forceinline__ void store(const Vals& r, T (*s)[LDS_LD], int tid) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int vi = tid + i * 256;
      int row = vi >> 3, kv = (vi & 7) * 8;
      *reinterpret_cast<V8*>(&s[row][kv]) = r.v[i];
    }
  }
};

// (k, n)-ordered operand: tile of 64 k x COLS n, n contiguous in memory.  Thread owns 4(k) x 8(n)
// micro-blocks: kq = lane % 16 (k0 = 4*kq), nv = wave*4 + lane/16 (+16 per pass).  Written to LDS
// transposed as [n][k] with 8-byte stores; with kq fastest across lanes those stores run at full
// LDS rate.
template <typename T, int COLS>
struct KnStage {
  static constexpr int NP = COLS / 128;
  using V8 = typename TypeTraits<T>::vec8;
  struct Vals { V8 v[NP][4]; };
  const T* p[NP];
  int64_t ld;
  int nvalid[NP];                           // columns of this thread's vector that exist (0..8)

  __device__ __forceinline__ void init(const T* base, int64_t ld_, int col0, int ncols, int tid, bool vec_ok) {
    int lane = tid & 63, wave = tid >> 6;
    int kq = lane & 15;
    ld = ld_;
#pragma unroll
    for (int ps = 0; ps < NP; ++ps) {
      int nv = wave * 4 + (lane >> 4) + ps * 16;
      int gn = col0 + nv * 8;
      nvalid[ps] = max(0, min(8, ncols - gn));
      if (vec_ok) gn = min(gn, ncols - 8);   // clamp to the last whole vector (ncols % 8 == 0 here)
      else gn = min(gn, ncols - 1);
      p[ps] = base + (int64_t)(kq * 4) * ld + gn;
    }
  }
  __device__ __forceinline__ void load_vec(Vals& r, int k0) const {
#pragma unroll
    for (int ps = 0; ps < NP; ++ps)
#pragma unroll
      for (int i = 0; i < 4; ++i) r.v[ps][i] = ldg16<V8>(p[ps] + (int64_t)(k0 + i) * ld);
  }
  __device__ __forceinline__ void load(Vals& r, int k0, int K, bool vec_ok, int tid) const {
    if (vec_ok && k0 + BK <= K) {
#pragma unroll
      for (int ps = 0; ps < NP; ++ps)
#pragma unroll
        for (int i = 0; i < 4; ++i) r.v[ps][i] = ldg16<V8>(p[ps] + (int64_t)(k0 + i) * ld);
      return;
    }
    int kq = tid & 15;
#pragma unroll
    for (int ps = 0; ps < NP; ++ps)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int gk = k0 + kq * 4 + i;
        V8 val;
#pragma unroll
        for (int e = 0; e < 8; ++e) val[e] = (T)0.0f;
        if (gk < K) {
          const T* q = p[ps] + (int64_t)(k0 + i) * ld;
          if (vec_ok) val = ldg16<V8>(q);
          else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (e < nvalid[ps]) val[e] = q[e];
          }
        }
        r.v[ps][i] = val;
      }
  }
  __device__ __forceinline__ void store(const Vals& r, T (*s)[LDS_LD], int tid) const {
    int lane = tid & 63, wave = tid >> 6;
    int kq = lane & 15;
#pragma unroll
    for (int ps = 0; ps < NP; ++ps) {
      int nv = wave * 4 + (lane >> 4) + ps * 16;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        typename TypeTraits<T>::vec4 w;
        w[0] = r.v[ps][0][e]; w[1] = r.v[ps][1][e]; w[2] = r.v[ps][2][e]; w[3] = r.v[ps][3][e];
        *reinterpret_cast<typename TypeTraits<T>::vec4*>(&s[nv * 8 + e][kq * 4]) = w;
      }
    }
  }
};

__device__ __forceinline__ int64_t epi_offset(const GemmArgs& g, int bt, int m, int n) {
  if (g.epi == EPI_MONARCH_SCATTER) {
    int dst_blk = n / g.per, j = n - dst_blk * g.per;
    return (int64_t)dst_blk * g.sL + (int64_t)m * g.ldc + (int64_t)bt * g.per + j;
  }
  return (int64_t)bt * g.sC + (int64_t)m * g.ldc + (int64_t)n * g.cn;
}

// Fused output stage (kernels instantiated with EP): bias (indexed by the element's offset inside its row of C) and
// activation are applied to the rounded result on its way out, like the separate kernels of the callers would.  The
// plain instantiations do not contain this code: it costs registers that the main loops need.
template <typename T>
__device__ __forceinline__ T ep_value(const GemmArgs& g, T r, int64_t in_row, int row) {
  float v = TypeTraits<T>::to_f32(r);
  if (g.bias) v += TypeTraits<T>::to_f32(reinterpret_cast<const T*>(g.bias)[in_row]);
  v = apply_act(v, g.act);
  if (g.gate || g.resid) {
    v = TypeTraits<T>::to_f32(TypeTraits<T>::from_f32(v));                    // what a separate gate / residual kernel would read
    if (g.gate) v *= TypeTraits<T>::to_f32(reinterpret_cast<const T*>(g.gate)[(int64_t)(row / g.gate_rows) * g.ld_gate + in_row]);
    if (g.resid) v += TypeTraits<T>::to_f32(reinterpret_cast<const T*>(g.resid)[(int64_t)row * g.ld_resid + in_row]);
  }
  return TypeTraits<T>::from_f32(v);
}

// eight consecutive outputs; their offset inside the row is a multiple of 8, so the bias comes as one 16-byte load
template <typename T>
__device__ __forceinline__ typename TypeTraits<T>::vec8 ep_vector(const GemmArgs& g, typename TypeTraits<T>::vec8 r, int64_t in_row, int row) {
  using V8 = typename TypeTraits<T>::vec8;
  V8 bv;
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = (T)0.0f;
  if (g.bias) bv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(g.bias) + in_row);
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = TypeTraits<T>::from_f32(apply_act(TypeTraits<T>::to_f32(r[e]) + TypeTraits<T>::to_f32(bv[e]), g.act));
  if (g.gate || g.resid) {                      // one row of gate per group of gate_rows rows of C
    V8 gv, rv;
#pragma unroll
    for (int e = 0; e < 8; ++e) { gv[e] = (T)1.0f; rv[e] = (T)0.0f; }
    if (g.gate) gv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(g.gate) + (int64_t)(row / g.gate_rows) * g.ld_gate + in_row);
    if (g.resid) rv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(g.resid) + (int64_t)row * g.ld_resid + in_row);
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = TypeTraits<T>::from_f32(TypeTraits<T>::to_f32(r[e]) * TypeTraits<T>::to_f32(gv[e]) + TypeTraits<T>::to_f32(rv[e]));
  }
  return r;
}

// Second tile of a pair: (r + bias) rounded to T, times the first tile's result, which the same thread stored at `c` before.
template <typename T>
__device__ __forceinline__ typename TypeTraits<T>::vec8 ep_pair_up(const GemmArgs& g, typename TypeTraits<T>::vec8 r, int64_t in_row, const T* c) {
  using V8 = typename TypeTraits<T>::vec8;
  V8 bv;
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = (T)0.0f;
  if (g.bias) bv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(g.bias) + in_row);
  const V8 gv = *reinterpret_cast<const V8*>(c);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const T up = TypeTraits<T>::from_f32(TypeTraits<T>::to_f32(r[e]) + TypeTraits<T>::to_f32(bv[e]));
    r[e] = TypeTraits<T>::from_f32(TypeTraits<T>::to_f32(gv[e]) * TypeTraits<T>::to_f32(up));
  }
  return r;
}

template <typename T, int BM, int BN, bool B_KN, int PD, bool EP = false>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmArgs g, int tiles_m, int tiles_n, int a_vec, int b_vec, int c_vec,
                                                        int per_xcd, int group_m) {
  constexpr int WM = BM / 2, WN = BN / 2;      // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;    // 32x32 MFMA tiles per wave
  using V8 = typename TypeTraits<T>::vec8;
  using Smem = GemmSmem<T, BM, BN>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem* sm = reinterpret_cast<Smem*>(smem_raw);  // two stages

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // Tile order.  Workgroups are handed to the 8 XCDs round-robin by linear id and each XCD has its own
  // L2, so the linear id is first turned into u = (id % 8) * per_xcd + id / 8: an XCD then works through a
  // contiguous range of u.  u walks the tiles of a batch entry in strips of group_m row tiles, column by
  // column, so the ~32 tiles an XCD has in flight form a roughly square patch of C and share their A and
  // B tiles through that XCD's L2 instead of every XCD fetching every weight tile.
  const int tiles = tiles_m * tiles_n;
  int u = blockIdx.x;
  if (per_xcd > 0) u = (u & 7) * per_xcd + (u >> 3);
  if (u >= tiles * g.batch) return;
  // interleaved columns: the batches of one tile write into the same cache lines, so they run next to each other
  const int bt = g.cn != 1 ? u % g.batch : u / tiles;
  const int ut = g.cn != 1 ? u / g.batch : u - bt * tiles;
  const int strip = ut / (group_m * tiles_n);
  const int rem = ut - strip * group_m * tiles_n;
  const int gm_here = min(group_m, tiles_m - strip * group_m);
  const int tm_i = strip * group_m + rem % gm_here, tn_i = rem / gm_here;
  const int m0 = tm_i * BM, n0 = tn_i * BN;

  const T* A = reinterpret_cast<const T*>(g.A) + (int64_t)bt * g.sA;
  const T* B = reinterpret_cast<const T*>(g.B) + (int64_t)bt * g.sB;
  T* C = reinterpret_cast<T*>(g.C);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  KcStage<T, BM> sa;
  KcStage<T, BN> sb_kc;
  KnStage<T, BN> sb_kn;
  // PD register sets of staged tiles: in the main loop the global loads run PD k-tiles ahead of the
  // multiplication.  Every load of that loop is unconditional (tile indices past the end are clamped
  // to the last full tile and fetched again for nothing), because a load under a condition makes the
  // number of loads in flight unknown to the compiler, which then waits for all of them.
  typename KcStage<T, BM>::Vals ra[PD];
  typename KcStage<T, BN>::Vals rb_kc[B_KN ? 1 : PD];
  typename KnStage<T, BN>::Vals rb_kn[B_KN ? PD : 1];

  const int KT = (g.K + BK - 1) / BK;
  const int KTm = (a_vec && b_vec) ? g.K / BK : 0;          // full tiles of 16-byte friendly operands
  sa.init(A, g.lda, m0, g.M, tid);
  if (B_KN) sb_kn.init(B, g.ldb, n0, g.N, tid, b_vec);
  else sb_kc.init(B, g.ldb, n0, g.N, tid);
  auto load_vec = [&](int d, int t) {
    sa.load_vec(ra[d], t * BK);
    if (B_KN) sb_kn.load_vec(rb_kn[B_KN ? d : 0], t * BK);
    else sb_kc.load_vec(rb_kc[B_KN ? 0 : d], t * BK);
  };
  auto store_tile = [&](int d, Smem& dst) {
    sa.store(ra[d], dst.a, tid);
    if (B_KN) sb_kn.store(rb_kn[B_KN ? d : 0], dst.b, tid);
    else sb_kc.store(rb_kc[B_KN ? 0 : d], dst.b, tid);
  };
  auto multiply = [&](Smem& cur) {
    // fragments of step kk + 1 are fetched from LDS before the matrix instructions of step kk are issued
    V8 af[2][TM], bf[2][TN];
    auto frags = [&](int kk, int set) {
      const int kof = kk * 16 + (lane >> 5) * 8;
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[set][i] = *reinterpret_cast<const V8*>(&cur.a[wm * WM + i * 32 + (lane & 31)][kof]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[set][j] = *reinterpret_cast<const V8*>(&cur.b[wn * WN + j * 32 + (lane & 31)][kof]);
    };
    frags(0, 0);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      if (kk + 1 < BK / 16) frags(kk + 1, (kk + 1) & 1);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = TypeTraits<T>::mfma32(af[kk & 1][i], bf[kk & 1][j], acc[i][j]);
    }
  };
  // one step of the pipelined loop; d (which register set is free) is a constant after unrolling
  auto step = [&](int kt, int d) {
    load_vec(d, min(kt + PD, KTm - 1));                      // set d went to LDS one step ago
    __builtin_amdgcn_sched_barrier(0);                       // keep the loads up here: the scheduler would sink them to their use
    multiply(sm[kt & 1]);
    store_tile((d + 1) % PD, sm[(kt + 1) & 1]);              // nobody reads that stage until the barrier
    __syncthreads();
  };
  int kt = 0;
  if (KTm > 0) {
#pragma unroll
    for (int d = 0; d < PD; ++d) load_vec(d, min(d, KTm - 1));
    store_tile(0, sm[0]);
    __syncthreads();
    for (; kt + PD <= KTm; kt += PD) {
#pragma unroll
      for (int d = 0; d < PD; ++d) step(kt + d, d);
    }
#pragma unroll
    for (int d = 0; d < PD - 1; ++d)
      if (kt + d < KTm) step(kt + d, d);
    kt = KTm;
  }
  // what the pipelined loop does not take - a partial last tile, or every tile of operands that are
  // not 16-byte friendly - goes one tile at a time through the guarded loads
  for (; kt < KT; ++kt) {
    sa.load(ra[0], kt * BK, g.K, a_vec, tid);
    if (B_KN) sb_kn.load(rb_kn[0], kt * BK, g.K, b_vec, tid);
    else sb_kc.load(rb_kc[0], kt * BK, g.K, b_vec, tid);
    store_tile(0, sm[kt & 1]);
    __syncthreads();
    multiply(sm[kt & 1]);
  }
  __syncthreads();                                             // the epilogue reuses the LDS tiles

  // D fragment: element e of lane l is row (e/4)*8 + (l/32)*4 + e%4, column l%32.
  if (c_vec) {
    // Stage the tile in LDS as [row][BN + 8] and write 16-byte row segments.
    constexpr int CLD = BN + 8;
    T* cs = reinterpret_cast<T*>(smem_raw);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        int col = wn * WN + j * 32 + (lane & 31);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          int row = wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          cs[row * CLD + col] = TypeTraits<T>::from_f32(g.sat8 ? sat8_rne(acc[i][j][e]) : acc[i][j][e]);
        }
      }
    __syncthreads();
    constexpr int VPR = BN / 8;                // 16-byte vectors per tile row
    for (int v = tid; v < BM * VPR; v += 256) {
      int row = v / VPR, cvec = (v - row * VPR) * 8;
      int gr = m0 + row, gc = n0 + cvec;
      if (gr < g.M && gc < g.N) {
        V8 v = *reinterpret_cast<const V8*>(&cs[row * CLD + cvec]);
        if (EP) v = ep_vector<T>(g, v, (int64_t)bt * g.sC + gc, gr);
        *reinterpret_cast<V8*>(&C[(int64_t)bt * g.sC + (int64_t)gr * g.ldc + gc]) = v;
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        int row = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row < g.M && col < g.N) {
          const int64_t off = epi_offset(g, bt, row, col);
          T v = TypeTraits<T>::from_f32(g.sat8 ? sat8_rne(acc[i][j][e]) : acc[i][j][e]);
          if (EP) v = ep_value<T>(g, v, off - (int64_t)row * g.ldc, row);
          C[off] = v;
        }
      }
    }
}

// ---- large problems: operand tiles copied global -> LDS without passing through registers --------------------------
// One workgroup per BM x BN tile: 4 waves as 2 x 2 (256 x 256: wave tile 128 x 128, 256 accumulator registers), or 8
// waves, two per SIMD, as 2 x 4 (256 x 256: wave tile 128 x 64) - the pair on a SIMD fills each other's waits at the
// barrier and for LDS, which is worth ~4 % on long reductions although a wave then reads 0.75 instead of 0.5 fragments
// per matrix instruction.  The k loop advances in
// stages of 32: a stage of A (BM rows x 64 bytes) and a stage of B live in two rings in LDS (4 and 5 stages), filled by
// global_load_lds_dwordx4 - each wave instruction moves 1 KiB and lane l's 16 bytes land at the wave's LDS address
// + 16 l, so the layout in LDS is chosen by which global address every lane fetches:
//   K-contiguous operand: chunk c (16 bytes) of row r sits at chunk position c ^ ((r >> 1) & 3), which makes the
//     128-bit fragment reads of 8 consecutive rows hit 8 different 16-byte bank groups;
//   (k, n) operand: 32 rows of BN n as they are in memory, chunk c of row k at position c ^ ((k & 3) << 1); the
//     fragments (8 consecutive k for one n) come out of ds_read_b64_tr_b16, which hands lane j of a 16-lane group
//     the j-th 16-bit column of the 4 rows whose addresses lanes 4e + j/4 supply.
// The loads are written as assembly so that the compiler does not count them: it would otherwise wait for all of them
// before every LDS read that follows.  The kernel waits itself (s_waitcnt vmcnt) before a stage is read.
// Ring depths.  SHALLOW (256x128, 128x128) keeps three stages of each operand instead of four and five, so that two
// (three) workgroups share a compute unit (72 KB / 48 KB each) and one's tile start-up and write-out run under the other's main loop:
// better when a compute unit gets several tiles with short reductions, worse when it gets one long one.
template <bool SHALLOW> constexpr int ring_na() { return SHALLOW ? 3 : 4; }
template <bool SHALLOW> constexpr int ring_nb() { return SHALLOW ? 3 : 5; }
template <int BM, int BN, bool SHALLOW>
constexpr size_t ring_lds_bytes() {
  size_t st = (size_t)(ring_na<SHALLOW>() * BM + ring_nb<SHALLOW>() * BN) * 64, ep = (size_t)BM * (BN + 8) * 2;
  return st > ep ? st : ep;
}

#ifdef BLR_TRACE
__device__ unsigned long long g_trace_gemm[4096 * 8];
#define TRG(i) do { if (threadIdx.x == 0 && blockIdx.x < 4096) g_trace_gemm[blockIdx.x * 8 + (i)] = wall_clock64(); } while (0)
#else
#define TRG(i) do {} while (0)
#endif

// The tile's way out of a ring kernel: accumulators -> LDS (as T, the stages are done with) -> whole rows to memory, through the
// output stage where there is one.  acc[i][j][4 q + e] is row (lane & 31), column 8 q + 4 (lane >> 5) + e of the 32 x 32 block
// (i, j) of the wave's WM x WN part (the products were formed transposed).  hf: which tile of a pair this is.
template <typename T, int BM, int BN, int BNC, int NWV, int WM, int WN, int TM, int TN, bool EP, bool PAIRS>
__device__ __forceinline__ void ring_write_out(const GemmArgs& g, f32x16 (&acc)[TM][TN], unsigned char* smem, T* C, int m0, int n0, int wm, int wn,
                                               int bt, int hf) {
  using V8 = typename TypeTraits<T>::vec8;
  const int tid = threadIdx.x, lane = tid & 63;
  __syncthreads();                                                   // the epilogue reuses the tile memory

  constexpr int CLD = BN + 8;
  T* cs = reinterpret_cast<T*>(smem);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wm * WM + i * 32 + (lane & 31);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wn * WN + j * 32 + q * 8 + (lane >> 5) * 4;
        typename TypeTraits<T>::vec4 v4;
#pragma unroll
        for (int e = 0; e < 4; ++e) v4[e] = TypeTraits<T>::from_f32(g.sat8 ? sat8_rne(acc[i][j][4 * q + e]) : acc[i][j][4 * q + e]);
        *reinterpret_cast<typename TypeTraits<T>::vec4*>(&cs[row * CLD + col]) = v4;
      }
    }
  __syncthreads();
  TRG(3);
  if (g.cn != 1) {
    // interleaved columns (column n of batch bt is element n * cn + bt of the row): two-byte stores, lanes along n, so
    // that an instruction touches cn * 128 contiguous bytes; the other batches fill the gaps
    for (int v = tid; v < BM * BNC; v += NWV * 64) {
      const int row = v / BNC, col = v - row * BNC;
      const int gr = m0 + row, gc = n0 + col;
      if (gr < g.M && gc < g.N) C[(int64_t)bt * g.sC + (int64_t)gr * g.ldc + (int64_t)gc * g.cn] = cs[row * CLD + col];
    }
    return;
  }
  constexpr int VPR = BNC / 8;
  for (int v = tid; v < BM * VPR; v += NWV * 64) {
    const int row = v / VPR, cvec = (v - row * VPR) * 8;
    const int gr = m0 + row, gc = n0 + cvec;
    if (gr < g.M && gc < g.N) {
      V8 v = *reinterpret_cast<const V8*>(&cs[row * CLD + cvec]);
      if (EP) {
        // (a pair: the first tile leaves silu(. + bias) where the result goes; the second is multiplied onto it by the thread that
        // stored it - the same element index v in both passes)
        if (!PAIRS || hf == 0) v = ep_vector<T>(g, v, (int64_t)bt * g.sC + gc, gr);
        else v = ep_pair_up<T>(g, v, (int64_t)bt * g.sC + gc + g.pair_dbias, &C[(int64_t)bt * g.sC + (int64_t)gr * g.ldc + gc]);
      }
      if (g.epi == EPI_MONARCH_SCATTER) {            // column c of entry bt -> block c / per, column bt * per + c % per
        const int d = gc / g.per;
        *reinterpret_cast<V8*>(&C[(int64_t)d * g.sL + (int64_t)gr * g.ldc + (int64_t)bt * g.per + (gc - d * g.per)]) = v;
      } else {
        *reinterpret_cast<V8*>(&C[(int64_t)bt * g.sC + (int64_t)gr * g.ldc + gc]) = v;
      }
    }
  }
}

// BNC: the columns of a tile that are computed and written.  Below BN (96 of 128) the stages keep their 128-column layout and the
// four waves sit above each other, 64 rows x 96 columns each: for output widths like 288 that 128-column tiles cover with a
// quarter of their matrix instructions wasted.
template <typename T, bool B_KN, int BM, int BN, bool EP = false, bool SHALLOW = false, int NWV = 4, bool PARTIAL = false, int BNC = BN>
__global__ __launch_bounds__(NWV * 64, (SHALLOW ? 2 : 1)) void gemm_ring_kernel(GemmArgs g, int tiles_m, int tiles_n, int per_xcd, int group_m, int side_wgs) {
  constexpr int NA = ring_na<SHALLOW>(), NB = ring_nb<SHALLOW>();
  constexpr int ASTG = BM * 64, BSTG = BN * 64, BRING = NA * ASTG;   // stage sizes, start of the B ring
  static_assert(BNC == BN || (BNC == 96 && BN == 128 && NWV == 4), "narrow tiles: 96 of 128 columns on four waves");
  constexpr int WGN = BNC != BN ? 1 : (NWV == 8 && BN == 256) ? 4 : 2, WGM = NWV / WGN;   // waves: 2 x 2, or 2 x 4 / 4 x 2 (two per SIMD), or 4 x 1
  constexpr int WM = BM / WGM, WN = BNC / WGN, TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / (16 * NWV), LB = BN / (16 * NWV);   // 1 KiB direct loads per wave and k tile
  constexpr int LT = LA + LB;
  constexpr int RB = BN * 2, CPR = BN / 8, RPI = 1024 / RB;
  constexpr int NMF = TM * TN;
  constexpr int SLOTS_PRE = NMF + NMF / 2;              // slots before the barrier of a step
  using V8 = typename TypeTraits<T>::vec8;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int tiles = tiles_m * tiles_n;
  TRG(0);
  int u = blockIdx.x;
  if (side_wgs > 0) {                                // the first workgroups of the launch carry the side job, not a tile (behind the
    if (u < side_wgs) {                              // tiles, in the tail of the launch, they measured 2 % of a DiT-XL/2 forward slower)
      for (int64_t idx = (int64_t)u * (NWV * 64) + tid; idx < g.side.items; idx += (int64_t)side_wgs * (NWV * 64)) side_prep_item<T>(g.side, idx);
      return;
    }
    u -= side_wgs;
  }
  if (per_xcd > 0) u = (u & 7) * per_xcd + (u >> 3);
  if (u >= tiles * g.batch) return;
  // interleaved columns: the batches of one tile write into the same cache lines, so they run next to each other (same
  // XCD, same time) and the lines are complete before they leave the L2
  const int bt = g.cn != 1 ? u % g.batch : u / tiles;
  const int ut = g.cn != 1 ? u / g.batch : u - bt * tiles;
  const int strip = ut / (group_m * tiles_n);
  const int rem = ut - strip * group_m * tiles_n;
  const int gm_here = min(group_m, tiles_m - strip * group_m);
  const int tm_i = strip * group_m + rem % gm_here, tn_i = rem / gm_here;
  const int m0 = tm_i * BM, n0 = tn_i * BNC;

  const char* Ab0 = reinterpret_cast<const char*>(g.A) + (int64_t)bt * g.sA * 2;
  const char* Bb0 = reinterpret_cast<const char*>(g.B) + (int64_t)bt * g.sB * 2;
  T* C = reinterpret_cast<T*>(g.C);
  // A pair of tiles (kernels with an output stage only): the second runs the same code on operands pair_dA / pair_dB further on
  // (not the 256 x 256 tile on four waves: it has no register left for the loop)
  constexpr bool PAIRS = EP && !PARTIAL && !(BM == 256 && BN == 256 && NWV == 4);
  const int halves = (PAIRS && g.pair) ? 2 : 1;
  for (int hf = 0; hf < halves; ++hf) {
  const char* Ab = Ab0 + (PAIRS ? (int64_t)hf * g.pair_dA * 2 : 0);
  const char* Bb = Bb0 + (PAIRS ? (int64_t)hf * g.pair_dB * 2 : 0);

  // PARTIAL: the batch index counts slices of the reduction (g.kc values of k each, the last one what is left of g.K)
  const int Kloc = PARTIAL ? min(g.kc, g.K - bt * g.kc) : g.K;
  const int KT = (Kloc + 31) >> 5;
  const int ktail = Kloc & 31;                        // valid k of the last tile when it is partial: 8, 16 or 24

  // K-contiguous operand tile: rows of 32 k (64 bytes); chunk c of row r is stored at chunk c ^ ((r >> 1) & 3).
  // (k, n) operand tile: 32 rows of BN n; chunk c of row k is stored at chunk c ^ ((k & 3) << 1): the four rows a
  // 16-lane group of a transposing read touches then sit in four different 32-byte bank groups.
  uint32_t a_off[LA], b_off[LB];
  const int row16 = lane >> 2;
  const int kc_chunk = (lane & 3) ^ ((row16 >> 1) & 3);
#pragma unroll
  for (int i = 0; i < LA; ++i)
    a_off[i] = (uint32_t)(min(m0 + (i * NWV + wave) * 16 + row16, g.M - 1) * g.lda * 2 + kc_chunk * 16);
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    if (B_KN) {
      const int krow = (i * NWV + wave) * RPI + lane / CPR;
      const int chunk = (lane % CPR) ^ ((krow & 3) << 1);
      b_off[i] = (uint32_t)(krow * g.ldb * 2 + min(n0 + chunk * 8, g.N - 8) * 2);
    } else {
      b_off[i] = (uint32_t)(min(n0 + (i * NWV + wave) * 16 + row16, g.N - 1) * g.ldb * 2 + kc_chunk * 16);
    }
  }
  // what to subtract from those offsets in a partial last tile (ktail valid k): the chunks of a K-contiguous row and the
  // rows of a (k, n) tile past ktail are replaced by valid ones (what lands there is multiplied by zeros)
  const int cmax = max((ktail >> 3) - 1, 0), rmax = max(ktail - 1, 0);
  const uint32_t tail_kc = (uint32_t)((kc_chunk - min(kc_chunk, cmax)) * 16);
  uint32_t tail_kn[LB];
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    const int krow = (i * NWV + wave) * RPI + lane / CPR;
    tail_kn[i] = B_KN ? (uint32_t)((krow - min(krow, rmax)) * g.ldb * 2) : tail_kc;
  }
  const uint32_t lds0 = ring_lds_addr(smem + wave * 1024);
  // load number li of the A tile ta (into A stage sa) or of the B tile tb (into B stage sb)
  auto issue_a = [&](int li, int ta, int sa, bool partial) {
    ring_load_lds(Ab + (int64_t)ta * 64, a_off[li] - (partial ? tail_kc : 0u), lds0 + sa * ASTG + li * (NWV * 1024));
  };
  auto issue_b = [&](int li, int tb, int sb, bool partial) {
    const char* Bp = B_KN ? Bb + (int64_t)tb * 32 * g.ldb * 2 : Bb + (int64_t)tb * 64;
    ring_load_lds(Bp, b_off[li] - (partial ? tail_kn[li] : 0u), lds0 + BRING + sb * BSTG + li * (NWV * 1024));
  };

  // fragment addresses
  const int half = lane >> 5;
  uint32_t rowA[TM], rowB[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) rowA[i] = (uint32_t)((wm * WM + i * 32 + (lane & 31)) * 64);
  const int g4 = lane >> 4, i16 = lane & 15;
  if (B_KN) {
    const int chunk0 = wn * WN / 8 + (g4 & 1) * 2 + ((i16 & 3) >> 1);
    const int swz = (i16 >> 2) << 1;
    const uint32_t kn_base = (uint32_t)(((g4 >> 1) * 8 + (i16 >> 2)) * RB + (i16 & 1) * 8);
#pragma unroll
    for (int j = 0; j < TN; ++j) rowB[j] = kn_base + (uint32_t)(((chunk0 + 4 * j) ^ swz) << 4);
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) rowB[j] = (uint32_t)((wn * WN + j * 32 + (lane & 31)) * 64);
  }
  uint32_t xo[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) xo[kk] = (uint32_t)((((kk * 2 + half) ^ ((lane >> 1) & 3)) << 4));

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  V8 af[2][TM], bf[2][TN];
  auto frags = [&](int sa, int sb, int kk, int set) {
    const unsigned char* sta = smem + sa * ASTG;
    const unsigned char* st = smem + BRING + sb * BSTG;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[set][i] = *reinterpret_cast<const V8*>(sta + rowA[i] + xo[kk]);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (B_KN) {
        union { V8 v; s16x4 h[2]; } w;
        w.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (kk * 16) * RB));
        w.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (kk * 16 + 4) * RB));
        bf[set][j] = w.v;
      } else {
        bf[set][j] = *reinterpret_cast<const V8*>(st + rowB[j] + xo[kk]);
      }
    }
  };
  auto mfma_one = [&](int set, int idx) {
    // the operands are handed over swapped, so that a product comes out transposed: lane l then holds, for row l & 31 of the
    // 32 x 32 block, four runs of four CONSECUTIVE columns (8 q + 4 (l >> 5) + 0..3, q = 0..3) - the write-out packs a run into
    // one 8-byte LDS store (one 16-byte store of partial sums) instead of four two-byte ones
    const int i = idx / TN, j = idx % TN;
    acc[i][j] = TypeTraits<T>::mfma32(bf[set][j], af[set][i], acc[i][j]);
  };

  // One k tile per step.  During step t the loads of A tile t + NA - 1 and of B tile t + NB - 1 go out (A first), into the
  // stages that tile t - 1 occupied.  Loads complete in the order they were issued, so "tile t + 1 has landed" is a bound
  // on the loads still in flight: everything issued after A(t+1) may be - that is B(t+NB-2) of the same step and the A and
  // B loads of the NA - 2 steps after it, this step included.  On entry set 0 holds the kk = 0 fragments of tile t.  The
  // loop body is one straight block for every tile: the last step also waits for, and fetches fragments of, a tile that
  // does not exist (whatever the stage holds; never multiplied), and a partial last tile multiplies what it lacks with
  // zeros.
  // With rings of equal depth B(t+1) goes out in the same step as A(t+1), after it: then only the loads of the NB - 2
  // later steps may be in flight.
  constexpr int INFLIGHT = NB > NA ? LB + (NA - 2) * LT : (NB - 2) * LT;
  static_assert(NB >= NA, "B must not be needed before A under the in-order bound");
#pragma unroll
  for (int s = 0; s < NB - 1; ++s) {
    const int tc = min(s, KT - 1);
    const bool partial = ktail && tc == KT - 1;
    if (s < NA - 1) {
#pragma unroll
      for (int li = 0; li < LA; ++li) issue_a(li, tc, s, partial);
    }
#pragma unroll
    for (int li = 0; li < LB; ++li) issue_b(li, tc, s, partial);
  }
  // in flight after A(0), B(0): A(1..NA-2), B(1..NB-2)
  __builtin_amdgcn_s_waitcnt(ring_vmcnt((NA - 2) * LA + (NB - 2) * LB));
  __builtin_amdgcn_s_barrier();
  TRG(1);
  frags(0, 0, 0, 0);
  int ca = 0, cb = 0;                                // stages of tile t in the two rings
  for (int t = 0; t < KT; ++t) {
    const int ta = min(t + NA - 1, KT - 1), tb = min(t + NB - 1, KT - 1);
    const bool pa = ktail && ta == KT - 1, pb = ktail && tb == KT - 1;
    const bool last_partial = ktail && t == KT - 1;
    const int sla = ca == 0 ? NA - 1 : ca - 1;
    const int slb = cb == 0 ? NB - 1 : cb - 1;
    frags(ca, cb, 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    // the step's loads go out between its first SLOTS_PRE matrix instructions, all of them before the barrier
    auto slot = [&](int sidx) {
      if (sidx < SLOTS_PRE && (sidx * LT) / SLOTS_PRE != ((sidx + 1) * LT) / SLOTS_PRE) {
        const int li = (sidx * LT) / SLOTS_PRE;
        __builtin_amdgcn_sched_barrier(0);
        if (li < LA) issue_a(li, ta, sla, pa);
        else issue_b(li - LA, tb, slb, pb);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // partial last tile: a lane's A fragment of slice kk covers k = (2 kk + half) * 8 .. + 7; those past ktail become zero
    if (last_partial && half * 8 >= ktail) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) af[0][i][e] = (T)0.0f;
    }
#pragma unroll
    for (int m = 0; m < NMF; ++m) { mfma_one(0, m); slot(m); }
    __builtin_amdgcn_sched_barrier(0);
    if (last_partial && (2 + half) * 8 >= ktail) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) af[1][i][e] = (T)0.0f;
    }
#pragma unroll
    for (int m = 0; m < NMF / 2; ++m) { mfma_one(1, m); slot(NMF + m); }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(ring_vmcnt(INFLIGHT));  // tile t + 1 has landed (this wave's part)
    __builtin_amdgcn_s_barrier();                    // everybody's part has, and nobody reads the stages of tile t any more
    ca = ca + 1 == NA ? 0 : ca + 1;
    cb = cb + 1 == NB ? 0 : cb + 1;
    frags(ca, cb, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = NMF / 2; m < NMF; ++m) mfma_one(1, m);
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
  TRG(2);
  if (PARTIAL) {
    // fp32 partial sums of this slice, straight from the accumulators: 16 bytes per lane (N is a multiple of 8, so a run of
    // four columns is inside or outside as a whole)
    float* P = reinterpret_cast<float*>(g.C) + (int64_t)bt * g.sC;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int gr = m0 + wm * WM + i * 32 + (lane & 31);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int gc = n0 + wn * WN + j * 32 + q * 8 + (lane >> 5) * 4;
          if (gr < g.M && gc < g.N)
            *reinterpret_cast<f32x4*>(&P[(int64_t)gr * g.ldc + gc]) = f32x4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        }
      }
    return;
  }
  ring_write_out<T, BM, BN, BNC, NWV, WM, WN, TM, TN, EP, PAIRS>(g, acc, smem, C, m0, n0, wm, wn, bt, hf);
  if (hf + 1 < halves) __syncthreads();              // the staged tile has been read: the rings may be filled again
  }  // tiles of a pair
  TRG(4);
}


// ---- the same kernel with operand stages of 64 k ---------------------------------------------------------------------------
// The vector memory path moves whole 128-byte lines from the L2: a load instruction that takes 64 bytes from each of 16 rows of
// a K-contiguous operand (a stage of 32 k) gets half of what it could - measured with every workgroup of the chip reading from
// an L2-resident buffer: 18-20 TB/s for 16 rows x 64 bytes per instruction against 35-37 TB/s for 8 rows x 128 bytes.  Here a
// stage is 64 k: an instruction takes the 128 bytes (eight 16-byte chunks) of each of 8 rows, lanes 8 r .. 8 r + 7 on row r, and
// lane (r, s) fetches chunk s ^ r, so that chunk c of row r lies at position c ^ (r & 7) of the row's 128 bytes in LDS: the
// fragment reads of eight consecutive rows (same chunk) then cover all banks.  A (k, n) operand stage is 64 rows of BN n, laid out
// as above.  NST stages (two or three) of both operands form one ring with one barrier per step of 64 k; a step is four sub-steps
// of 16 k (one fragment of each 32-row block).
// What the loop is made of, per step of a 256 x 256 tile on eight waves (two per SIMD): 64 matrix instructions per SIMD (2048
// cycles of its matrix pipe), 192 KiB of fragment reads (about 770 cycles of the LDS), 64 KiB of operand loads into LDS in 64 load
// instructions that queue in the compute unit's one address path.  In-kernel cycle counts: 2890 cycles per step with the fragment reads of a sub-step issued as one burst ahead of its
// products and the barrier at the end of the step, 2570 with one read or load between two products and the barrier between the
// third and the fourth sub-step (behind it a wave still holds a sub-step of products in registers, under which the first fragments
// of the next stage arrive).  The clock drops as the pipe fills up (1.35 -> 1.27 GHz under the board's power limit with random
// operands), so the second gain in cycles is worth 4 % in time.
template <int BM, int BN, int NST>
constexpr size_t ring64_lds_bytes() {
  size_t st = (size_t)NST * (BM + BN) * 128, ep = (size_t)BM * (BN + 8) * 2;
  return st > ep ? st : ep;
}

template <typename T, bool B_KN, int BM, int BN, bool EP, int NWV, int NST, int PER_CU, bool HALF = false>
__global__ __launch_bounds__(NWV * 64, (NWV / 4) * PER_CU) void gemm_ring64_kernel(GemmArgs g, int tiles_m, int tiles_n, int per_xcd, int group_m, int side_wgs) {
  constexpr int ASTG = BM * 128, BSTG = BN * 128, BRING = NST * ASTG;
  constexpr int WGN = (NWV == 8 && BN == 256) ? 4 : 2, WGM = NWV / WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / (8 * NWV), LB = BN / (8 * NWV), LT = LA + LB;     // 1 KiB loads per wave and stage
  constexpr int RB = BN * 2, CPR = BN / 8, RPI = 1024 / RB;                 // (k, n) operand: bytes per k row, chunks per row, rows per load
  constexpr int NMF = TM * TN;
  constexpr int SLOTS = NMF;                                                // matrix instructions between which a step's loads go out
  static_assert(NMF >= TM + TN, "a sub-step has a gap for every fragment read");
  static_assert(LA >= 1 && LB >= 1 && NST >= 2, "tile too small for the workgroup");
  using V8 = typename TypeTraits<T>::vec8;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int tiles = tiles_m * tiles_n;
  TRG(0);
  int u = blockIdx.x;
  if (side_wgs > 0) {
    if (u < side_wgs) {
      for (int64_t idx = (int64_t)u * (NWV * 64) + tid; idx < g.side.items; idx += (int64_t)side_wgs * (NWV * 64)) side_prep_item<T>(g.side, idx);
      return;
    }
    u -= side_wgs;
  }
  if (per_xcd > 0) u = (u & 7) * per_xcd + (u >> 3);
  if (u >= tiles * g.batch) return;
  const int bt = u / tiles;
  const int ut = u - bt * tiles;
  const int strip = ut / (group_m * tiles_n);
  const int rem = ut - strip * group_m * tiles_n;
  const int gm_here = min(group_m, tiles_m - strip * group_m);
  const int tm_i = strip * group_m + rem % gm_here, tn_i = rem / gm_here;
  const int m0 = tm_i * BM, n0 = tn_i * BN;

  const char* Ab0 = reinterpret_cast<const char*>(g.A) + (int64_t)bt * g.sA * 2;
  const char* Bb0 = reinterpret_cast<const char*>(g.B) + (int64_t)bt * g.sB * 2;
  T* C = reinterpret_cast<T*>(g.C);
  constexpr bool PAIRS = EP && !(BM == 256 && BN == 256 && NWV == 4);
  const int halves = (PAIRS && g.pair) ? 2 : 1;
  for (int hf = 0; hf < halves; ++hf) {
  const char* Ab = Ab0 + (PAIRS ? (int64_t)hf * g.pair_dA * 2 : 0);
  const char* Bb = Bb0 + (PAIRS ? (int64_t)hf * g.pair_dB * 2 : 0);

  const int KT = (g.K + 63) >> 6;
  const int ktail = g.K & 63;                         // valid k of the last stage when it is partial: a multiple of 8

  // lane (r8, s8) of a K-contiguous load: row r8 of the instruction's eight, LDS position s8 of its 128 bytes, global chunk s8 ^ r8
  const int r8 = lane >> 3, s8 = lane & 7, c8 = s8 ^ r8;
  uint32_t a_off[LA], b_off[LB];
#pragma unroll
  for (int i = 0; i < LA; ++i) a_off[i] = (uint32_t)(min(m0 + (i * NWV + wave) * 8 + r8, g.M - 1) * g.lda * 2 + c8 * 16);
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    if (B_KN) {
      const int krow = (i * NWV + wave) * RPI + lane / CPR;
      const int chunk = (lane % CPR) ^ ((krow & 3) << 1);
      b_off[i] = (uint32_t)(krow * g.ldb * 2 + min(n0 + chunk * 8, g.N - 8) * 2);
    } else {
      b_off[i] = (uint32_t)(min(n0 + (i * NWV + wave) * 8 + r8, g.N - 1) * g.ldb * 2 + c8 * 16);
    }
  }
  // a partial last stage: chunks (rows of a (k, n) stage) past ktail are replaced by valid ones; what lands there meets zeros
  const int cmax = max((ktail >> 3) - 1, 0), rmax = max(ktail - 1, 0);
  const uint32_t tail_kc = (uint32_t)((c8 - min(c8, cmax)) * 16);
  uint32_t tail_kn[LB];
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    const int krow = (i * NWV + wave) * RPI + lane / CPR;
    tail_kn[i] = B_KN ? (uint32_t)((krow - min(krow, rmax)) * g.ldb * 2) : tail_kc;
  }
  const uint32_t lds0 = ring_lds_addr(smem + wave * 1024);
  // HALF (eight waves, two stages, no clamped row of either K-contiguous operand, no partial stage: the launcher checks): a stage's loads cannot
  // be spread over the step here, and every wave that issues one waits in the compute unit's address path while its SIMD's other
  // wave may be waiting there too.  Waves 0..3 - one per SIMD - therefore issue the loads of waves 4..7 as well: those rows lie
  // NWV / 2 load instructions further down, a wave-uniform offset, so the same per-lane offsets serve (no row is clamped; the column clamp of a (k, n) operand belongs to the lane and is the same for both).
  static_assert(!HALF || (NWV == 8 && NST == 2), "the one configuration this is for");
  constexpr int ISS = HALF ? 2 : 1;
  const bool issuer = !HALF || wave < NWV / 2;
  const int64_t dA = (int64_t)(NWV / 2) * 8 * g.lda * 2;
  const int64_t dB = B_KN ? (int64_t)(NWV / 2) * RPI * g.ldb * 2 : (int64_t)(NWV / 2) * 8 * g.ldb * 2;
  auto issue = [&](int li, int tile, int stg, bool partial) {       // load li (A first, then B) of stage `tile` into ring slot stg
    if (HALF && !issuer) return;                                     // (wave-uniform)
    if (li < LA) {
      ring_load_lds(Ab + (int64_t)tile * 128, a_off[li] - (partial ? tail_kc : 0u), lds0 + stg * ASTG + li * (NWV * 1024));
      if (HALF) ring_load_lds(Ab + (int64_t)tile * 128 + dA, a_off[li] - (partial ? tail_kc : 0u), lds0 + stg * ASTG + li * (NWV * 1024) + (NWV / 2) * 1024);
    } else {
      const int lb = li - LA;
      const char* Bp = B_KN ? Bb + (int64_t)tile * 64 * g.ldb * 2 : Bb + (int64_t)tile * 128;
      ring_load_lds(Bp, b_off[lb] - (partial ? tail_kn[lb] : 0u), lds0 + BRING + stg * BSTG + lb * (NWV * 1024));
      if (HALF) ring_load_lds(Bp + dB, b_off[lb] - (partial ? tail_kn[lb] : 0u), lds0 + BRING + stg * BSTG + lb * (NWV * 1024) + (NWV / 2) * 1024);
    }
  };

  // fragment addresses: row rl of a K-contiguous stage starts at (rl >> 3) KiB + (rl & 7) * 128; sub-step q, lane half h wants
  // chunk 2 q + h, which lies at position (2 q + h) ^ (rl & 7), and rl & 7 = lane & 7
  const int half = lane >> 5;
  uint32_t rowA[TM], rowB[TN], xo[4];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int rl = wm * WM + i * 32 + (lane & 31);
    rowA[i] = (uint32_t)(((rl >> 3) << 10) + ((rl & 7) << 7));
  }
  const int g4 = lane >> 4, i16 = lane & 15;
  if (B_KN) {
    const int chunk0 = wn * WN / 8 + (g4 & 1) * 2 + ((i16 & 3) >> 1);
    const int swz = (i16 >> 2) << 1;
    const uint32_t kn_base = (uint32_t)(((g4 >> 1) * 8 + (i16 >> 2)) * RB + (i16 & 1) * 8);
#pragma unroll
    for (int j = 0; j < TN; ++j) rowB[j] = kn_base + (uint32_t)(((chunk0 + 4 * j) ^ swz) << 4);
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int rl = wn * WN + j * 32 + (lane & 31);
      rowB[j] = (uint32_t)(((rl >> 3) << 10) + ((rl & 7) << 7));
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) xo[q] = (uint32_t)(((2 * q + half) ^ (lane & 7)) << 4);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  V8 af[2][TM], bf[2][TN];
  auto frags = [&](int stg, int q, int set) {
    const unsigned char* sta = smem + stg * ASTG;
    const unsigned char* st = smem + BRING + stg * BSTG;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[set][i] = *reinterpret_cast<const V8*>(sta + rowA[i] + xo[q]);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (B_KN) {
        union { V8 v; s16x4 h[2]; } w;
        w.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (q * 16) * RB));
        w.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (q * 16 + 4) * RB));
        bf[set][j] = w.v;
      } else {
        bf[set][j] = *reinterpret_cast<const V8*>(st + rowB[j] + xo[q]);
      }
    }
  };
  // fragment number idx of a sub-step, in the order the products want them: A 0, all of B, the rest of A
  auto frag_one = [&](int stg, int q, int set, int idx) {
    const unsigned char* sta = smem + stg * ASTG;
    const unsigned char* st = smem + BRING + stg * BSTG;
    if (idx == 0 || idx > TN) {
      const int i = idx == 0 ? 0 : idx - TN;
      af[set][i] = *reinterpret_cast<const V8*>(sta + rowA[i] + xo[q]);
    } else {
      const int j = idx - 1;
      if (B_KN) {
        union { V8 v; s16x4 h[2]; } w;
        w.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (q * 16) * RB));
        w.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(st + rowB[j] + (q * 16 + 4) * RB));
        bf[set][j] = w.v;
      } else {
        bf[set][j] = *reinterpret_cast<const V8*>(st + rowB[j] + xo[q]);
      }
    }
  };
  auto mfma_one = [&](int set, int idx) {              // (operands swapped: the product comes out transposed, see the kernel above)
    const int i = idx / TN, j = idx % TN;
    acc[i][j] = TypeTraits<T>::mfma32(bf[set][j], af[set][i], acc[i][j]);
  };
  auto zero_tail = [&](int set, int q) {               // a partial last stage: the A fragment of chunk 2 q + half is past ktail
    if ((2 * q + half) * 8 >= ktail) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) af[set][i][e] = (T)0.0f;
    }
  };

  // All NST stages go out before the loop.  Step t: sub-steps 0, 1 and 2 run while the fragments of sub-steps 1, 2 and 3 are read;
  // once those are in registers nobody needs stage t in LDS any more, and that is where the step's one barrier stands.  The loads
  // of stage t + NST go out behind it, into the slot of stage t, between the products of sub-step 3.
#pragma unroll
  for (int s = 0; s < NST; ++s) {
    const int tc = min(s, KT - 1);
    const bool partial = ktail && tc == KT - 1;
#pragma unroll
    for (int li = 0; li < LT; ++li) issue(li, tc, s, partial);
  }
  __builtin_amdgcn_s_waitcnt(ring_vmcnt((NST - 1) * LT * ISS));
  __builtin_amdgcn_s_barrier();
  TRG(1);
  frags(0, 0, 0);
#ifdef BLR_TRACE
  uint64_t trw_v = 0, trw_b = 0;
  const uint64_t trw_0 = __builtin_amdgcn_s_memtime();
#endif
  int cs = 0;                                         // ring slot of stage t
  for (int t = 0; t < KT; ++t) {
    const int tn = min(t + NST, KT - 1);
    const bool pn = ktail && tn == KT - 1;
    const bool last_partial = ktail && t == KT - 1;
    const int nq = last_partial ? (ktail + 15) >> 4 : 4;             // sub-steps with anything to add
    const int nx = cs + 1 == NST ? 0 : cs + 1;
    // With three stages the slot that the barrier of step t frees is needed only at the barrier of step t + 2, so its loads go out
    // over four sub-steps (part 0 in sub-step 3 of step t, parts 1..3 in sub-steps 0..2 of step t + 1) instead of queueing in the
    // compute unit's address path all at once; with two stages they must all go at once (part 0).
    constexpr int PARTS = NST >= 3 ? 4 : 1;
    const int tp = min(t - 1 + NST, KT - 1);                 // the stage whose later parts go out in this step, and its slot
    const bool pp = ktail && tp == KT - 1;
    const int sp = cs == 0 ? NST - 1 : cs - 1;
    auto slot = [&](int sidx, int part) {
      const int s2 = part * SLOTS + sidx;
      if (part < PARTS && (s2 * LT) / (PARTS * SLOTS) != ((s2 + 1) * LT) / (PARTS * SLOTS)) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int li = (s2 * LT) / (PARTS * SLOTS); li < ((s2 + 1) * LT) / (PARTS * SLOTS); ++li) {
          if (part == 0) issue(li, tn, cs, pn);
          else issue(li, tp, sp, pp);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // A sub-step: its products, between them - one per gap - the fragment reads of the next sub-step (a wave cannot issue a
    // product while it issues something else, and a burst of reads or loads leaves the matrix pipe idle when the SIMD's other wave
    // is in the same burst), and in the last sub-step the loads of stage t + NST.
    auto substep = [&](int set, bool live, int stg_next, int q_next, int part) {      // part: which part of a stage's loads goes with it
#pragma unroll
      for (int m = 0; m < NMF; ++m) {
        if (live) mfma_one(set, m);
        if (m < TM + TN) frag_one(stg_next, q_next, set ^ 1, m);
        slot(m, part);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    if (last_partial) zero_tail(0, 0);
    substep(0, true, cs, 1, 1);       // (in step 0 parts 1..3 repeat loads of the last stage the prologue asked for, into the same slot)
    if (last_partial) zero_tail(1, 1);
    substep(1, nq > 1, cs, 2, 2);
    if (last_partial) zero_tail(0, 2);
    substep(0, nq > 2, cs, 3, 3);
    // the step's barrier: stage t is in registers, stage t + 1 has landed
#ifdef BLR_TRACE
    const uint64_t tw0 = __builtin_amdgcn_s_memtime();
#endif
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_waitcnt(ring_vmcnt((NST - 2) * LT * ISS));   // (later stages may still be out)
#ifdef BLR_TRACE
    const uint64_t tw1 = __builtin_amdgcn_s_memtime();
#endif
    __builtin_amdgcn_s_barrier();
#ifdef BLR_TRACE
    const uint64_t tw2 = __builtin_amdgcn_s_memtime();
    trw_v += tw1 - tw0; trw_b += tw2 - tw1;
#endif
    __builtin_amdgcn_sched_barrier(0);
    if (last_partial) zero_tail(1, 3);
    substep(1, nq > 3, nx, 0, 0);
    cs = nx;
  }
  __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
  TRG(2);
#ifdef BLR_TRACE
  if (tid == 0 && blockIdx.x < 4096) {               // wave 0: cycles waiting for its loads, at the barrier, and in the whole loop
    g_trace_gemm[blockIdx.x * 8 + 5] = trw_v; g_trace_gemm[blockIdx.x * 8 + 6] = trw_b; g_trace_gemm[blockIdx.x * 8 + 7] = __builtin_amdgcn_s_memtime() - trw_0;
  }
#endif
  ring_write_out<T, BM, BN, BN, NWV, WM, WN, TM, TN, EP, PAIRS>(g, acc, smem, C, m0, n0, wm, wn, bt, hf);
  if (hf + 1 < halves) __syncthreads();
  }  // tiles of a pair
  TRG(4);
}

// ---- fp32 verification GEMM: 64x64 tile, 16x16 threads, 4x4 outputs per thread ---------------
template <bool B_KN>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs g, int tiles_m) {
  __shared__ float as[16][64 + 1];
  __shared__ float bs[16][64 + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int bt = blockIdx.y;
  const int m0 = (blockIdx.x % tiles_m) * 64, n0 = (blockIdx.x / tiles_m) * 64;
  const float* A = reinterpret_cast<const float*>(g.A) + (int64_t)bt * g.sA;
  const float* B = reinterpret_cast<const float*>(g.B) + (int64_t)bt * g.sB;
  float* C = reinterpret_cast<float*>(g.C);
  float acc[4][4] = {};
  for (int k0 = 0; k0 < g.K; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int idx = tid + i * 256;               // 0..1023
      {                                      // A tile: row = idx / 16, k = idx % 16
        int r = idx >> 4, k = idx & 15;
        int gr = m0 + r, gk = k0 + k;
        as[k][r] = (gr < g.M && gk < g.K) ? A[(int64_t)gr * g.lda + gk] : 0.0f;
      }
      if (B_KN) {                            // k = idx / 64, n = idx % 64
        int k = idx >> 6, n = idx & 63;
        int gk = k0 + k, gn = n0 + n;
        bs[k][n] = (gk < g.K && gn < g.N) ? B[(int64_t)gk * g.ldb + gn] : 0.0f;
      } else {                               // n = idx / 16, k = idx % 16
        int n = idx >> 4, k = idx & 15;
        int gk = k0 + k, gn = n0 + n;
        bs[k][n] = (gk < g.K && gn < g.N) ? B[(int64_t)gn * g.ldb + gk] : 0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { av[i] = as[k][ty * 4 + i]; bv[i] = bs[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int row = m0 + ty * 4 + i, col = n0 + tx * 4 + j;
      if (row < g.M && col < g.N) {
        const int64_t off = epi_offset(g, bt, row, col);
        float v = g.sat8 ? sat8_rne(acc[i][j]) : acc[i][j];
        if (g.bias || g.act || g.gate || g.resid) v = ep_value<float>(g, v, off - (int64_t)row * g.ldc, row);
        C[off] = v;
      }
    }
}

template <typename T, int BM, int BN, bool B_KN>
static void* mfma_kernel_ptr(bool ep) {          // (two k-tiles of global loads in flight: PD = 2)
  return ep ? (void*)gemm_mfma_kernel<T, BM, BN, B_KN, 2, true> : (void*)gemm_mfma_kernel<T, BM, BN, B_KN, 2>;
}

template <typename T, int BM, int BN>
static int launch_mfma(const GemmArgs& g, hipStream_t st) {
  int tiles_m = (int)cdiv(g.M, BM), tiles_n = (int)cdiv(g.N, BN);
  // 16-byte vector accesses need every row start and every k (or n) offset to be 16-byte aligned.
  int a_vec = aligned(g.A, 16) && g.lda % 8 == 0 && g.sA % 8 == 0;
  int b_vec = aligned(g.B, 16) && g.ldb % 8 == 0 && g.sB % 8 == 0;
  int c_vec = g.epi == EPI_PLAIN && g.cn == 1 && aligned(g.C, 16) && g.ldc % 8 == 0 && g.sC % 8 == 0 && g.N % 8 == 0 &&
              (!g.bias || aligned(g.bias, 16)) && (!g.gate || (aligned(g.gate, 16) && g.ld_gate % 8 == 0)) && (!g.resid || (aligned(g.resid, 16) && g.ld_resid % 8 == 0));
  size_t lds = 2 * sizeof(GemmSmem<T, BM, BN>);
  const bool ep = g.bias != nullptr || g.act != 0 || g.gate != nullptr || g.resid != nullptr;
  void* fn = g.b_kn ? mfma_kernel_ptr<T, BM, BN, true>(ep) : mfma_kernel_ptr<T, BM, BN, false>(ep);
  static std::mutex mu;
  static std::set<void*> raised;
  {
    std::lock_guard<std::mutex> lk(mu);
    if (lds > 64 * 1024 && !raised.count(fn)) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) { set_error("gemm: cannot raise LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
      raised.insert(fn);
    }
  }
  const int64_t total = (int64_t)tiles_m * tiles_n * g.batch;
  if (total > (1ll << 30)) { set_error("gemm: too many tiles"); return BLR_ERR_UNSUPPORTED; }
  int per_xcd = (int)cdiv(total, 8);
  int group_m = 4;
  dim3 grid((unsigned)(per_xcd > 0 ? per_xcd * 8 : total));
  GemmArgs ga = g;
  void* args[] = {&ga, &tiles_m, &tiles_n, &a_vec, &b_vec, &c_vec, &per_xcd, &group_m};
  hipError_t e = hipLaunchKernel(fn, grid, dim3(256), args, lds, st);
  if (e != hipSuccess) { set_error("gemm_mfma: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

// The ring kernels take plain row-major output and 16-byte friendly operands whose per-lane byte offsets fit 32 bits.
// out[m, n] = sum over slices s of P[s][m][n] (fp32, fixed order), rounded once to T; 8 columns per thread
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, T* __restrict__ C, int M, int N, int64_t ldc, int splits) {
  using V8 = typename TypeTraits<T>::vec8;
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int vpr = N >> 3;
  if (v >= (int64_t)M * vpr) return;
  const int m = (int)(v / vpr), n = (int)(v - (int64_t)m * vpr) * 8;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
  for (int s = 0; s < splits; ++s) {
    const float4* p = reinterpret_cast<const float4*>(P + ((int64_t)s * M + m) * N + n);
    const float4 a = p[0], b = p[1];
    acc[0] += a.x; acc[1] += a.y; acc[2] += a.z; acc[3] += a.w;
    acc[4] += b.x; acc[5] += b.y; acc[6] += b.z; acc[7] += b.w;
  }
  V8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32(acc[e]);
  *reinterpret_cast<V8*>(&C[(int64_t)m * ldc + n]) = o;
}

// How many slices a plain single GEMM is cut into along K: only when 256 x 128 tiles leave at least half of the compute
// units idle and every slice keeps at least 512 values of k (slices are multiples of 32).
static int splitk_plan(int M, int N, int K, int* kc_out) {
  const int cus = device_cus() > 0 ? device_cus() : 256;
  const int64_t tiles = cdiv(M, 256) * cdiv(N, 128);
  if (M < 96 || N % 8 || K % 8 || tiles * 2 > cus) return 1;
  int splits = (int)std::min<int64_t>(8, cus / tiles);
  while (splits > 1 && K / splits < 512) --splits;
  if (splits <= 1) return 1;
  const int kc = (int)cdiv(cdiv(K, splits), 32) * 32;
  splits = (int)cdiv(K, kc);
  if (kc_out) *kc_out = kc;
  return splits;
}

size_t gemm_splitk_bytes(int M, int N, int K, int dtype) {
  if (dtype != BLR_F16 && dtype != BLR_BF16) return 0;
  const int splits = splitk_plan(M, N, K, nullptr);
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

static bool ring_ok(const GemmArgs& g) {
  if (g.cn < 1 || g.N < 8 || g.N % 8 || g.K % 8) return false;
  // Monarch's scatter of the first product: an 8-column vector stays inside one destination block when the period is a multiple of 8
  if (g.epi == EPI_MONARCH_SCATTER && (g.per % 8 || g.sL % 8 || g.cn != 1 || g.sat8 || g.bias || g.act || g.gate || g.resid)) return false;
  if (g.epi != EPI_PLAIN && g.epi != EPI_MONARCH_SCATTER) return false;
  if (!aligned(g.A, 16) || !aligned(g.B, 16) || g.lda % 8 || g.sA % 8 || g.ldb % 8 || g.sB % 8) return false;
  if (g.cn == 1) {                                   // 16-byte stores, the fused output stage reads its vector the same way
    if (!aligned(g.C, 16) || (g.bias && !aligned(g.bias, 16)) || (g.gate && (!aligned(g.gate, 16) || g.ld_gate % 8)) || (g.resid && (!aligned(g.resid, 16) || g.ld_resid % 8)) || g.ldc % 8 || g.sC % 8) return false;
  } else if (g.bias || g.act || g.gate || g.resid) {
    return false;                                    // interleaved columns are stored one by one, without an output stage
  }
  const int64_t lim = (int64_t)1 << 32;
  if ((int64_t)(g.M - 1) * g.lda * 2 + 64 >= lim) return false;
  if (g.b_kn ? 31 * g.ldb * 2 + (int64_t)g.N * 2 >= lim : (int64_t)(g.N - 1) * g.ldb * 2 + 64 >= lim) return false;
  return true;
}

template <typename T, int BM, int BN, bool SHALLOW = false, int NWV = 4, bool PARTIAL = false, int BNC = BN>
static int launch_ring(const GemmArgs& g, hipStream_t st) {
  int tiles_m = (int)cdiv(g.M, BM), tiles_n = (int)cdiv(g.N, BNC);
  const size_t lds = ring_lds_bytes<BM, BN, SHALLOW>();
  const bool ep = g.bias != nullptr || g.act != 0 || g.gate != nullptr || g.resid != nullptr;
  void* fn;
  if constexpr (PARTIAL)
    fn = g.b_kn ? (void*)gemm_ring_kernel<T, true, BM, BN, false, SHALLOW, NWV, true> : (void*)gemm_ring_kernel<T, false, BM, BN, false, SHALLOW, NWV, true>;
  else
    fn = ep ? (g.b_kn ? (void*)gemm_ring_kernel<T, true, BM, BN, true, SHALLOW, NWV, false, BNC> : (void*)gemm_ring_kernel<T, false, BM, BN, true, SHALLOW, NWV, false, BNC>)
            : (g.b_kn ? (void*)gemm_ring_kernel<T, true, BM, BN, false, SHALLOW, NWV, false, BNC> : (void*)gemm_ring_kernel<T, false, BM, BN, false, SHALLOW, NWV, false, BNC>);
  static std::mutex mu;
  static std::set<void*> raised;
  {
    std::lock_guard<std::mutex> lk(mu);
    if (!raised.count(fn)) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) { set_error("gemm: cannot raise LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
      raised.insert(fn);
    }
  }
  const int64_t total = (int64_t)tiles_m * tiles_n * g.batch;
  if (total > (1ll << 30)) { set_error("gemm: too many tiles"); return BLR_ERR_UNSUPPORTED; }
  int per_xcd = (int)cdiv(total, 8);
  int group_m = 4;
  // a side job: one thread per item, in workgroups ahead of the tiles (a multiple of eight of them, so that tile u stays on XCD u % 8)
  int side_wgs = 0;
  if (!PARTIAL && g.side.items > 0 && g.side_taken) side_wgs = (int)(cdiv(cdiv(g.side.items, NWV * 64), 8) * 8);
  if (side_wgs > 4096) side_wgs = 4096;
  dim3 grid((unsigned)((per_xcd > 0 ? per_xcd * 8 : total) + side_wgs));
  GemmArgs ga = g;
  void* args[] = {&ga, &tiles_m, &tiles_n, &per_xcd, &group_m, &side_wgs};
  hipError_t e = hipLaunchKernel(fn, grid, dim3(NWV * 64), args, lds, st);
  if (e != hipSuccess) { set_error("gemm_ring: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  if (side_wgs > 0) *g.side_taken = 1;
  return BLR_OK;
}

template <typename T, int BM, int BN, int NWV, int NST, int PER_CU>
static int launch_ring64(const GemmArgs& g, hipStream_t st) {
  int tiles_m = (int)cdiv(g.M, BM), tiles_n = (int)cdiv(g.N, BN);
  const size_t lds = ring64_lds_bytes<BM, BN, NST>();
  const bool ep = g.bias != nullptr || g.act != 0 || g.gate != nullptr || g.resid != nullptr;
  void* fn = ep ? (g.b_kn ? (void*)gemm_ring64_kernel<T, true, BM, BN, true, NWV, NST, PER_CU> : (void*)gemm_ring64_kernel<T, false, BM, BN, true, NWV, NST, PER_CU>)
                : (g.b_kn ? (void*)gemm_ring64_kernel<T, true, BM, BN, false, NWV, NST, PER_CU> : (void*)gemm_ring64_kernel<T, false, BM, BN, false, NWV, NST, PER_CU>);
  if constexpr (NWV == 8 && NST == 2) {
    // no tile with a clamped row and no partial stage: four of the eight waves issue all loads (see the kernel).  A ragged last
    // column tile is fine with a (k, n) operand: its clamp is on the lane's column, the same in both halves of a stage's rows
    if (g.M % BM == 0 && (g.N % BN == 0 || (g.b_kn && g.N % 8 == 0)) && g.K % 64 == 0)
      fn = ep ? (g.b_kn ? (void*)gemm_ring64_kernel<T, true, BM, BN, true, NWV, NST, PER_CU, true> : (void*)gemm_ring64_kernel<T, false, BM, BN, true, NWV, NST, PER_CU, true>)
              : (g.b_kn ? (void*)gemm_ring64_kernel<T, true, BM, BN, false, NWV, NST, PER_CU, true> : (void*)gemm_ring64_kernel<T, false, BM, BN, false, NWV, NST, PER_CU, true>);
  }
  static std::mutex mu;
  static std::set<void*> raised;
  {
    std::lock_guard<std::mutex> lk(mu);
    if (!raised.count(fn)) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) { set_error("gemm: cannot raise LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
      raised.insert(fn);
    }
  }
  const int64_t total = (int64_t)tiles_m * tiles_n * g.batch;
  if (total > (1ll << 30)) { set_error("gemm: too many tiles"); return BLR_ERR_UNSUPPORTED; }
  int per_xcd = (int)cdiv(total, 8);
  int group_m = 4;
  int side_wgs = 0;
  if (g.side.items > 0 && g.side_taken) side_wgs = (int)(cdiv(cdiv(g.side.items, NWV * 64), 8) * 8);
  if (side_wgs > 4096) side_wgs = 4096;
  dim3 grid((unsigned)(per_xcd * 8 + side_wgs));
  GemmArgs ga = g;
  void* args[] = {&ga, &tiles_m, &tiles_n, &per_xcd, &group_m, &side_wgs};
  hipError_t e = hipLaunchKernel(fn, grid, dim3(NWV * 64), args, lds, st);
  if (e != hipSuccess) { set_error("gemm_ring64: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  if (side_wgs > 0) *g.side_taken = 1;
  return BLR_OK;
}

template <typename T>
static int pick_mfma(const GemmArgs& g, hipStream_t st) {
  // Bigger tiles do more MFMA work per LDS byte (the 2x2 wave grid reads 0.5 fragments per MFMA at
  // 256x256, 0.75 at 256x128, 1 at 128x128) but need enough tiles to fill the 256 CUs.
  const int cus = device_cus() > 0 ? device_cus() : 256;
  int64_t t256 = cdiv(g.M, 256) * cdiv(g.N, 256) * g.batch;
  int64_t t128 = cdiv(g.M, 256) * cdiv(g.N, 128) * g.batch;
  // Problems with enough work go to the ring kernels, with the largest of their tiles that still gives every compute unit
  // one (BLR_GEMM_RING: 0 never, 1 by this rule, 2 whenever the operands allow it; BLR_GEMM_RING_TILE = 256256, 256128
  // or 128128 picks the tile, BLR_GEMM_RING_PER_CU = 1 or 2 the deep or the shallow variant of the two smaller tiles,
  // BLR_GEMM_RING_WAVES = 4 or 8 the workgroup size of the two larger ones - options that tests switch with
  // blr_set_option).
  const int ring = option_value(OPT_GEMM_RING, 1);
  if (ring > 0 && ring_ok(g) && g.epi == EPI_PLAIN && g.splitk_ws && g.batch == 1 && g.cn == 1 && !g.sat8 && !g.bias && !g.act && !g.gate && !g.resid) {
    // few tiles, long reduction: slices of K as the batch of the partial-sum kernel, then one pass that adds them up
    int kc = 0;
    const int splits = option_value(OPT_GEMM_SPLITK, 1) == 0 ? 1 : splitk_plan(g.M, g.N, g.K, &kc);
    if (splits > 1 && g.splitk_bytes >= (size_t)splits * g.M * g.N * sizeof(float) && aligned(g.splitk_ws, 16)) {
      GemmArgs p = g;
      p.batch = splits; p.kc = kc;
      p.sA = kc; p.sB = g.b_kn ? (int64_t)kc * g.ldb : kc;
      p.C = g.splitk_ws; p.ldc = g.N; p.sC = (int64_t)g.M * g.N;
      int rc = launch_ring<T, 256, 128, false, 4, true>(p, st);
      if (rc) return rc;
      const int64_t vecs = (int64_t)g.M * (g.N / 8);
      hipLaunchKernelGGL((splitk_reduce_kernel<T>), dim3((unsigned)cdiv(vecs, 256)), dim3(256), 0, st,
                         reinterpret_cast<const float*>(g.splitk_ws), reinterpret_cast<T*>(g.C), g.M, g.N, g.ldc, splits);
      BLR_CHECK_LAUNCH("splitk_reduce");
      return BLR_OK;
    }
  }
  if (g.pair && (!ring_ok(g) || g.epi != EPI_PLAIN || g.cn != 1 || g.sat8 || g.gate || g.resid || g.pair_dA % 8 || g.pair_dB % 8 || g.pair_dbias % 8 || !aligned(g.C, 16))) {
    set_error("gemm: a pair of tiles (SiLU-gated halves) needs 16-byte aligned operands, K and the half width multiples of 8, a plain row-major output");
    return BLR_ERR_UNSUPPORTED;
  }
  if ((ring > 0 && ring_ok(g)) || g.pair) {
    int rt = option_value(OPT_GEMM_RING_TILE, 0);
    const bool auto_tile = rt == 0, narrow = rt == 256096;
    if (narrow) rt = 256128;
    const int64_t fill = ((int64_t)cus * 9 + 9) / 10;
    const int64_t r128 = cdiv(g.M, 128) * cdiv(g.N, 128) * g.batch;
    int per_cu = option_value(OPT_GEMM_RING_PER_CU, 0);
    bool wide64 = false;                       // a tile chosen together with stages of 64 k
    // interleaved columns are bound by their two-byte stores: only worth it with several tiles per compute unit
    if (rt == 0 && g.cn != 1 && ring < 2 && t128 < 2 * (int64_t)cus) rt = -1;
    if (rt == 0) {
      // short reductions are mostly tile start-up and write-out: two workgroups per compute unit overlap those
      // (a reduction of a few steps only: the smaller tile, three workgroups per compute unit - 4096 x 288 x 72 in 16 batches
      // 1.7 us faster than with 256 x 128)
      if (g.K <= 128 && r128 >= 3 * (int64_t)cus) { rt = 128128; if (!per_cu) per_cu = 2; }
      // a wide output with a reduction of a thousand or two: enough 256 x 256 tiles for two rounds, and the big tile's lower LDS
      // traffic per matrix instruction beats the overlap of two smaller workgroups (2048 x 22016 x 1024: 164.7 -> 154.1 us for
      // the whole low-rank call; four batches of 2048 x 5504 x 1024: Monarch 184.6 -> 176.8 us)
      else if (g.K >= 1024 && g.K <= 2048 && g.N >= 2048 && t256 >= 2 * (int64_t)cus) rt = 256256;
      // the same for batched products from a reduction of eight stages of 64 k, where 256-column tiles waste at most an eighth of
      // their columns: per-kernel times at 2048 rows, 16 batches: 1376 columns, K = 1024 (Z U of BLAST 4096 -> 22016) 118.0 -> 112.4 us,
      // 1024 columns, K = 688 (x V of 11008 -> 4096) 75.1 -> 66.8 us
      else if (g.cn == 1 && g.K >= 512 && g.K <= 2048 && g.N >= 1024 && cdiv(g.N, 256) * 256 * 8 <= (int64_t)g.N * 9 && t256 >= 2 * (int64_t)cus) { rt = 256256; wide64 = true; }
      else if (g.K <= 2048 && t128 >= 2 * (int64_t)cus) { rt = 256128; if (!per_cu) per_cu = 2; }
      // batched products from eight stages of 64 k that are exactly one round of 256 x 128 tiles: one such tile per compute unit on
      // 64-k stages rather than two workgroups of 128 x 128 (Z U of BLAST 4096 -> 4096 at 2048 rows, 16 x 2048 x 256 x 512: the call
      // 55.1 -> 52.8 us; 54.2 with 64-k stages on the 128 x 128 tiles)
      else if (g.batch > 1 && g.cn == 1 && g.K >= 512 && g.K < 1024 && t128 >= fill && t128 <= (int64_t)cus) { rt = 256128; wide64 = true; }
      else if (g.K <= 512 && r128 >= fill) rt = 128128;
      // a narrow output (one 128-column tile, mostly empty at 256): more, smaller tiles (4096 x 72 x 576 in 16 batches:
      // 26.8 us with 256 x 256 tiles, 20.7 with 256 x 128, 19.7 with 128 x 128)
      else if (g.N <= 128 && g.K <= 1024 && r128 >= fill) rt = 128128;
      else if (t256 >= fill) rt = 256256;
      else if (t128 >= fill) rt = 256128;
      else if (r128 >= fill || ring > 1 || g.pair) rt = 128128;
    }
    if (g.pair && rt <= 0) rt = 128128;
    if (rt > 0 && (ring > 1 || g.pair || (g.M >= 96 && g.K >= 64))) {
      // Stages of 64 k (plain row-major output only): by default for reductions of a thousand or more - single products, and
      // batched ones that give a compute unit at most two 256 x 128 tiles - and for the wide batched products that the rule above
      // gave 256 x 256 tiles.  Other batched products with many tiles per compute unit or short reductions (most of BLAST's) live
      // on two workgroups of 256 x 128 per compute unit overlapping each other's tile start-up and write-out, which the larger
      // stages leave no LDS for (2048 rows: dense 4096 -> 22016 355 -> 335 us, 11008 -> 4096 207 -> 174 us; BLAST 4096 -> 22016
      // 186 -> 201 us with every product on 64-k stages of 256 x 128 tiles, 186 -> 190 with only Z U (K = 1024, 1408 tiles), while
      // 11008 -> 4096, whose Z U has 256 tiles, gains: 139.3 -> 134.8 us; Monarch 4096 -> 4096 / 11008 -> 4096
      // 64.9 -> 61.8 / 96.3 -> 88.8 us, side by side on one box; DiT-XL/2 with dense layers 11.67 -> 11.04 ms, with BLAST layers 11.76 -> 12.25 ms when
      // forced).  BLR_GEMM_RING_BK = 32 / 64 decides for every problem.
      if (option_value(OPT_GEMM_RING_BK, wide64 || (g.K >= 1024 && (g.batch == 1 || t128 <= 2 * (int64_t)cus)) ? 64 : 32) == 64 && g.cn == 1) {
        const bool w8 = option_value(OPT_GEMM_RING_WAVES, 8) == 8;
        if (rt == 256256) return !w8 && !g.pair ? launch_ring64<T, 256, 256, 4, 2, 1>(g, st) : launch_ring64<T, 256, 256, 8, 2, 1>(g, st);
        if (rt == 256128) return w8 ? launch_ring64<T, 256, 128, 8, 3, 1>(g, st) : launch_ring64<T, 256, 128, 4, 3, 1>(g, st);
        return per_cu == 1 ? launch_ring64<T, 128, 128, 4, 3, 1>(g, st) : launch_ring64<T, 128, 128, 4, 2, 2>(g, st);
      }
      if (rt == 256256) {
        // eight waves (2 x 4, wave tile 128 x 64, two per SIMD) hide each other's barrier and LDS waits: the default
        return option_value(OPT_GEMM_RING_WAVES, 8) == 4 && !g.pair ? launch_ring<T, 256, 256>(g, st) : launch_ring<T, 256, 256, false, 8>(g, st);
      }
      if (rt == 256128) {
        if (per_cu != 2 && option_value(OPT_GEMM_RING_WAVES, 4) == 8) return launch_ring<T, 256, 128, false, 8>(g, st);
        // 96-column tiles where they cover the width with at most 4/5 of what 128-column tiles compute (288 = 3 x 96 against 3 x 128)
        // (BLR_GEMM_RING_TILE = 256096 asks for them, 256128 keeps them away)
        if (g.cn == 1 && (narrow || (auto_tile && per_cu == 2 && cdiv(g.N, 96) * 96 * 5 <= cdiv(g.N, 128) * 128 * 4)))
          return launch_ring<T, 256, 128, true, 4, false, 96>(g, st);
        return per_cu == 2 ? launch_ring<T, 256, 128, true>(g, st) : launch_ring<T, 256, 128>(g, st);
      }
      if (!per_cu) per_cu = r128 >= 2 * (int64_t)cus ? 2 : 1;     // three shallow workgroups per compute unit, or two deep ones
      return per_cu == 2 ? launch_ring<T, 128, 128, true>(g, st) : launch_ring<T, 128, 128>(g, st);
    }
  }
  // short reductions are dominated by filling and draining a tile: two smaller workgroups per CU overlap those
  if (g.M >= 256 && t128 >= cus && g.K > 1024) return launch_mfma<T, 256, 128>(g, st);
  return launch_mfma<T, 128, 128>(g, st);
}

int gemm_launch(const GemmArgs& g, int dtype, hipStream_t st) {
  if (g.M <= 0 || g.N <= 0 || g.K <= 0 || g.batch <= 0) { set_error("gemm: empty problem"); return BLR_ERR_BAD_ARG; }
  // A handful of rows is a weight-streaming problem, not a tiling problem: plain products with (k, n)-ordered weights go to
  // the slab kernel of the decode path (it declines what it cannot take, e.g. a reduction deeper than one slab here).
  if (g.M <= 16 && g.b_kn && g.cn == 1 && g.epi == EPI_PLAIN && !g.sat8 && !g.bias && g.act == 0 && !g.gate && !g.resid && (dtype == BLR_F16 || dtype == BLR_BF16)) {
    int rc = slab_gemm_launch(g.A, g.lda, g.sA, g.B, g.ldb, g.sB, g.C, g.ldc, g.sC, g.M, g.N, g.K, g.batch, dtype, nullptr, 1, st);
    if (rc != 1) return rc;
  }
  if (dtype == BLR_F16) return pick_mfma<f16>(g, st);
  if (dtype == BLR_BF16) return pick_mfma<bf16>(g, st);
  if (dtype == BLR_F32) {
    int tiles_m = (int)cdiv(g.M, 64), tiles_n = (int)cdiv(g.N, 64);
    dim3 grid(tiles_m * tiles_n, g.batch);
    if (g.b_kn) hipLaunchKernelGGL((gemm_f32_kernel<true>), grid, dim3(256), 0, st, g, tiles_m);
    else hipLaunchKernelGGL((gemm_f32_kernel<false>), grid, dim3(256), 0, st, g, tiles_m);
    BLR_CHECK_LAUNCH("gemm_f32");
    return BLR_OK;
  }
  set_error("gemm: unknown dtype %d", dtype);
  return BLR_ERR_BAD_ARG;
}

// ---- BLAST rank-space mix ------------------------------------------------------------------
// Workgroup = (64-wide r chunk) x (32 rows of m per pass); the S slab S(:, :, r chunk) is staged
// in LDS as fp32 [j][i][64] once per workgroup and reused for every m pass.
template <typename T, int MAXB>
__global__ __launch_bounds__(256) void blast_mix_kernel(const T* __restrict__ Y, const T* __restrict__ S,
                                                        T* __restrict__ Z, int M, int b, int R,
                                                        int64_t s_si, int64_t s_sj, int64_t s_sr, int m_per_wg, int sat8) {
  extern __shared__ float s_lds[];           // [b][b][64]  (j, i, r)
  const int tid = threadIdx.x;
  const int r0 = blockIdx.x * 64;
  const int rr = tid & 63, ms = tid >> 6;    // 64 r lanes x 4 m slots
  for (int idx = tid; idx < b * b * 64; idx += 256) {
    int r = idx & 63, ji = idx >> 6;
    int j = ji / b, i = ji - j * b;
    float v = 0.0f;
    if (r0 + r < R) v = TypeTraits<T>::to_f32(S[(int64_t)i * s_si + (int64_t)j * s_sj + (int64_t)(r0 + r) * s_sr]);
    s_lds[idx] = v;
  }
  __syncthreads();
  const int r = r0 + rr;
  if (r >= R) return;
  const int m_begin = blockIdx.y * m_per_wg;
  const int m_end = min(M, m_begin + m_per_wg);
  for (int m = m_begin + ms; m < m_end; m += 4) {
    if (MAXB > 0) {                          // b <= MAXB: every Y value is loaded once
      float yv[MAXB > 0 ? MAXB : 1];
#pragma unroll
      for (int j = 0; j < MAXB; ++j) yv[j] = (j < b) ? TypeTraits<T>::to_f32(Y[((int64_t)j * M + m) * R + r]) : 0.0f;
      for (int i = 0; i < b; ++i) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXB; ++j)
          if (j < b) acc = fmaf(s_lds[(j * b + i) * 64 + rr], yv[j], acc);
        Z[((int64_t)i * M + m) * R + r] = TypeTraits<T>::from_f32(sat8 ? sat8_rne(acc) : acc);
      }
    } else {
      for (int i = 0; i < b; ++i) {
        float acc = 0.0f;
        for (int j = 0; j < b; ++j)
          acc = fmaf(s_lds[(j * b + i) * 64 + rr], TypeTraits<T>::to_f32(Y[((int64_t)j * M + m) * R + r]), acc);
        Z[((int64_t)i * M + m) * R + r] = TypeTraits<T>::from_f32(sat8 ? sat8_rne(acc) : acc);
      }
    }
  }
}

template <typename T>
static void mix_dispatch(dim3 grid, size_t lds, hipStream_t st, const void* Y, const void* S, void* Z, int M, int b, int R,
                         int64_t s_si, int64_t s_sj, int64_t s_sr, int m_per_wg, int sat8) {
  if (b <= 16)
    hipLaunchKernelGGL((blast_mix_kernel<T, 16>), grid, dim3(256), lds, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, sat8);
  else
    hipLaunchKernelGGL((blast_mix_kernel<T, 0>), grid, dim3(256), lds, st, (const T*)Y, (const T*)S, (T*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, sat8);
}

// S slab of a workgroup of the mix kernels: s_t[(j * b + i) * MIX_LDR + r] = S(i, j, r0 + r) for 64 ranks, zero past R.  Rows
// of 72 elements, not 64: staging S stored (r, i, j) writes one (j, i) row per lane, and with rows of 128 bytes every lane of a
// wave would hit the same bank (the mix of a 4608 -> 1152, rank 576 layer at 4096 rows took 54 us with S in that order and
// 40 us with S (j, i, r); 16-byte reads of a row stay aligned with 144-byte rows).
constexpr int MIX_LDR = 72;
// 16-byte pieces along whichever of r or j is contiguous in memory; element-wise otherwise.
template <typename T>
__device__ __forceinline__ void mix_stage_s(const T* __restrict__ S, T* s_t, int b, int R, int r0,
                                            int64_t s_si, int64_t s_sj, int64_t s_sr, int vec_ok) {
  using V8 = typename TypeTraits<T>::vec8;
  const int tid = threadIdx.x;
  if (vec_ok && s_sr == 1) {                                   // (j, i, r) or (i, j, r): r contiguous
    for (int idx = tid; idx < b * b * 8; idx += 256) {
      const int r8 = (idx & 7) * 8, ji = idx >> 3;
      const int j = ji / b, i = ji - j * b;
      V8 v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (T)0.0f;
      if (r0 + r8 < R) v = *reinterpret_cast<const V8*>(&S[(int64_t)i * s_si + (int64_t)j * s_sj + r0 + r8]);
      *reinterpret_cast<V8*>(&s_t[ji * MIX_LDR + r8]) = v;
    }
  } else if (vec_ok && s_sj == 1 && (b & 7) == 0) {            // (r, i, j): j contiguous
    const int jv = b >> 3;
    for (int idx = tid; idx < 64 * b * jv; idx += 256) {
      const int j8 = (idx % jv) * 8, t = idx / jv;
      const int i = t % b, r = t / b;
      V8 v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (T)0.0f;
      if (r0 + r < R) v = *reinterpret_cast<const V8*>(&S[(int64_t)(r0 + r) * s_sr + (int64_t)i * s_si + j8]);
#pragma unroll
      for (int e = 0; e < 8; ++e) s_t[((j8 + e) * b + i) * MIX_LDR + r] = v[e];
    }
  } else {
    for (int idx = tid; idx < b * b * 64; idx += 256) {
      const int r = idx & 63, ji = idx >> 6;
      const int j = ji / b, i = ji - j * b;
      T v = (T)0.0f;
      if (r0 + r < R) v = S[(int64_t)i * s_si + (int64_t)j * s_sj + (int64_t)(r0 + r) * s_sr];
      s_t[ji * MIX_LDR + r] = v;
    }
  }
}

// Vector variant for two-byte types, b <= 16, R % 8 == 0: thread = (8 consecutive r, one m); all
// b vectors Y_j[m, r..r+7] are loaded (16 bytes each) before the b x b x 8 multiply-adds, S comes
// from an LDS slab [j][i][64] staged once per workgroup and reused for 128 rows of m.
template <typename T>
__global__ __launch_bounds__(256) void blast_mix_vec_kernel(const T* __restrict__ Y, const T* __restrict__ S,
                                                            T* __restrict__ Z, int M, int b, int R,
                                                            int64_t s_si, int64_t s_sj, int64_t s_sr, int m_per_wg, int s_vec, int sat8) {
  using V8 = typename TypeTraits<T>::vec8;
  extern __shared__ float s_lds[];
  T* s_t = reinterpret_cast<T*>(s_lds);      // [b][b][64]  (j, i, r)
  const int tid = threadIdx.x;
  const int r0 = blockIdx.x * 64;
  mix_stage_s<T>(S, s_t, b, R, r0, s_si, s_sj, s_sr, s_vec);
  __syncthreads();
  const int rl = tid & 7, ms = tid >> 3;     // 8 r-vectors x 32 m slots
  const int r = r0 + rl * 8;
  if (r >= R) return;
  const int m_begin = blockIdx.y * m_per_wg;
  const int m_end = min(M, m_begin + m_per_wg);
  for (int m = m_begin + ms; m < m_end; m += 32) {
    V8 yv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j)                     // unconditional: planes past b re-read the last one and are not used
      yv[j] = ldg16<V8>(&Y[((int64_t)min(j, b - 1) * M + m) * R + r]);
    for (int i = 0; i < b; ++i) {
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if (j < b) {
          V8 sv = *reinterpret_cast<const V8*>(&s_t[(j * b + i) * MIX_LDR + rl * 8]);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = fmaf(TypeTraits<T>::to_f32(sv[e]), TypeTraits<T>::to_f32(yv[j][e]), acc[e]);
        }
      }
      V8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32(sat8 ? sat8_rne(acc[e]) : acc[e]);
      *reinterpret_cast<V8*>(&Z[((int64_t)i * M + m) * R + r]) = o;
    }
  }
}

// fp16 only: the same mix with packed half-precision multiply-adds (two per lane and instruction).
// The b <= 16 products of one output are accumulated in fp16; Z is stored as fp16 anyway and the
// reference rounds it to 16 bits as well, so this costs about one extra rounding of the result.
template <bool FULL16, int MB>                   // FULL16: b == 16, so no load sits under a condition; MB rows of m per thread
__global__ __launch_bounds__(256) void blast_mix_h2_kernel(const f16* __restrict__ Y, const f16* __restrict__ S,
                                                           f16* __restrict__ Z, int M, int b, int R,
                                                           int64_t s_si, int64_t s_sj, int64_t s_sr, int m_per_wg, int s_vec) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  struct H8 { h2 v[4]; };
  extern __shared__ float s_lds[];
  f16* s_t = reinterpret_cast<f16*>(s_lds);      // [b][b][64]  (j, i, r)
  const int tid = threadIdx.x;
  const int r0 = blockIdx.x * 64;
  mix_stage_s<f16>(S, s_t, b, R, r0, s_si, s_sj, s_sr, s_vec);
  __syncthreads();
  const int rl = tid & 7, ms = tid >> 3;     // 8 r-vectors x 32 m slots
  const int r = r0 + rl * 8;
  if (r >= R) return;
  const int m_begin = blockIdx.y * m_per_wg;
  const int m_end = min(M, m_begin + m_per_wg);
  // Each S vector read from LDS serves MB rows: the kernel is otherwise bound by LDS reads (16 bytes per 8 multiply-adds).
  for (int m = m_begin + ms; m < m_end; m += 32 * MB) {
    H8 yv[MB][16];
#pragma unroll
    for (int u = 0; u < MB; ++u) {
      const int mu = min(m + 32 * u, M - 1);         // rows past the end are fetched again and not stored
#pragma unroll
      for (int j = 0; j < 16; ++j)                   // unconditional: planes past b re-read the last one and are not used
        yv[u][j] = *reinterpret_cast<const H8*>(&Y[((int64_t)(FULL16 ? j : min(j, b - 1)) * M + mu) * R + r]);
    }
    for (int i = 0; i < b; ++i) {
      H8 acc[MB];
#pragma unroll
      for (int u = 0; u < MB; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[u].v[e] = h2{(_Float16)0.0f, (_Float16)0.0f};
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if (FULL16 || j < b) {
          const H8 sv = *reinterpret_cast<const H8*>(&s_t[(j * b + i) * MIX_LDR + rl * 8]);
#pragma unroll
          for (int u = 0; u < MB; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[u].v[e] = sv.v[e] * yv[u][j].v[e] + acc[u].v[e];
        }
      }
#pragma unroll
      for (int u = 0; u < MB; ++u)
        if (m + 32 * u < m_end) *reinterpret_cast<H8*>(&Z[((int64_t)i * M + m + 32 * u) * R + r]) = acc[u];
    }
  }
}

// The mix for a handful of rows (M <= 16, b <= 16): workgroup = 16 ranks x all output blocks, thread = (block i, rank).
// The Y values of the chunk (b x M x 16) are staged in LDS once; every thread keeps its b values of S in registers.
template <typename T>
__global__ __launch_bounds__(256) void blast_mix_small_kernel(const T* __restrict__ Y, const T* __restrict__ S, T* __restrict__ Z,
                                                              int M, int b, int R, int64_t s_si, int64_t s_sj, int64_t s_sr) {
  __shared__ float ys[16 * 16 * 16];                  // [j][m][rank in chunk]
  const int tid = threadIdx.x, g = tid >> 4, rr = tid & 15;
  const int r0 = blockIdx.x * 16, r = r0 + rr;
  float sv[16];
#pragma unroll
  for (int j = 0; j < 16; ++j)
    sv[j] = (g < b && j < b && r < R) ? TypeTraits<T>::to_f32(S[(int64_t)g * s_si + (int64_t)j * s_sj + (int64_t)r * s_sr]) : 0.0f;
  const int total = b * M * 16;
  for (int idx = tid; idx < total; idx += 256) {
    const int c = idx & 15, jm = idx >> 4;            // jm = j * M + m
    ys[idx] = (r0 + c < R) ? TypeTraits<T>::to_f32(Y[(int64_t)jm * R + r0 + c]) : 0.0f;
  }
  __syncthreads();
  if (g < b && r < R) {
    for (int m = 0; m < M; ++m) {
      float z = 0.0f;
#pragma unroll
      for (int j = 0; j < 16; ++j) z = fmaf(sv[j], j < b ? ys[(j * M + m) * 16 + rr] : 0.0f, z);
      Z[((int64_t)g * M + m) * R + r] = TypeTraits<T>::from_f32(z);
    }
  }
}

int blast_mix_launch(const void* Y, const void* S, void* Z, int M, int b, int R,
                     int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype, hipStream_t st, int sat8) {
  if (M <= 16 && b <= 16 && !sat8 && (dtype == BLR_F16 || dtype == BLR_BF16)) {
    const dim3 grid((unsigned)cdiv(R, 16));
    if (dtype == BLR_F16) hipLaunchKernelGGL(blast_mix_small_kernel<f16>, grid, dim3(256), 0, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr);
    else hipLaunchKernelGGL(blast_mix_small_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)Y, (const bf16*)S, (bf16*)Z, M, b, R, s_si, s_sj, s_sr);
    BLR_CHECK_LAUNCH("blast_mix_small");
    return BLR_OK;
  }
  int r_chunks = (int)cdiv(R, 64);
  if (dtype != BLR_F32 && b <= 16 && R % 8 == 0 && aligned(Y, 16) && aligned(Z, 16)) {
    size_t lds = (size_t)b * b * MIX_LDR * 2;
    // S may be fetched in 16-byte pieces if every piece starts on a 16-byte boundary
    const int s_vec = aligned(S, 16) && ((s_sr == 1 && s_si % 8 == 0 && s_sj % 8 == 0) ||
                                         (s_sj == 1 && s_si % 8 == 0 && s_sr % 8 == 0));
    const bool use_h2 = dtype == BLR_F16 && !sat8;
    const int mb = use_h2 && M >= 64 ? 2 : 1;
    int m_per_wg = 32 * mb;                        // one pass of the 32 row slots: more, smaller workgroups measured fastest
    dim3 grid(r_chunks, (unsigned)cdiv(M, m_per_wg));
    if (use_h2 && mb == 2)
      if (b == 16) hipLaunchKernelGGL((blast_mix_h2_kernel<true, 2>), grid, dim3(256), lds, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec);
      else hipLaunchKernelGGL((blast_mix_h2_kernel<false, 2>), grid, dim3(256), lds, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec);
    else if (use_h2)
      if (b == 16) hipLaunchKernelGGL((blast_mix_h2_kernel<true, 1>), grid, dim3(256), lds, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec);
      else hipLaunchKernelGGL((blast_mix_h2_kernel<false, 1>), grid, dim3(256), lds, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec);
    else if (dtype == BLR_F16)
      hipLaunchKernelGGL(blast_mix_vec_kernel<f16>, grid, dim3(256), lds, st, (const f16*)Y, (const f16*)S, (f16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec, sat8);
    else
      hipLaunchKernelGGL(blast_mix_vec_kernel<bf16>, grid, dim3(256), lds, st, (const bf16*)Y, (const bf16*)S, (bf16*)Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, s_vec, sat8);
    BLR_CHECK_LAUNCH("blast_mix_vec");
    return BLR_OK;
  }
  size_t lds = (size_t)b * b * 64 * sizeof(float);
  if (lds > 64 * 1024) { set_error("blast mix: b=%d too large for the LDS slab", b); return BLR_ERR_UNSUPPORTED; }
  int m_per_wg = 64;
  while ((int64_t)r_chunks * cdiv(M, m_per_wg) < 1024 && m_per_wg > 4) m_per_wg /= 2;
  dim3 grid(r_chunks, (unsigned)cdiv(M, m_per_wg));
  if (dtype == BLR_F16) mix_dispatch<f16>(grid, lds, st, Y, S, Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, sat8);
  else if (dtype == BLR_BF16) mix_dispatch<bf16>(grid, lds, st, Y, S, Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, sat8);
  else mix_dispatch<float>(grid, lds, st, Y, S, Z, M, b, R, s_si, s_sj, s_sr, m_per_wg, sat8);
  BLR_CHECK_LAUNCH("blast_mix");
  return BLR_OK;
}

}  // namespace blr

// ---- matrix-core probe ----------------------------------------------------------------------------------------------
// What the matrix cores sustain with nothing in their way: one workgroup of eight waves per compute unit, every wave a chain of
// eight independent 32x32x16 products per iteration, operands in registers.  With `random` the operands are pseudo-random
// numbers in [-2, 2) instead of ones (the power drawn, and with it the clock, depends on the data); with `lds_reads` every group
// of eight products is accompanied by that many 1 KiB fragment reads from LDS (6 = what a 128 x 64 wave tile needs).
namespace blr {
template <bool RANDOM, int READS>
__global__ __launch_bounds__(512) void mfma_probe_kernel(unsigned* sink, int iters) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[32768];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 32768 / 4; i += 512) reinterpret_cast<unsigned*>(smem)[i] = i;
  __syncthreads();
  f32x16 acc[8];
#pragma unroll
  for (int a = 0; a < 8; ++a)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[a][e] = 0.f;
  f16x8 fa = {1, 1, 1, 1, 1, 1, 1, 1}, fb = fa;
  if (RANDOM) {
    unsigned h = (tid * 2654435761u) ^ (blockIdx.x * 40503u) ^ 0x9e3779b9u;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h ^= h << 13; h ^= h >> 17; h ^= h << 5;
      fa[e] = (f16)(((int)(h & 0xffff) - 32768) / 16384.0f);
      h ^= h << 13; h ^= h >> 17; h ^= h << 5;
      fb[e] = (f16)(((int)(h & 0xffff) - 32768) / 16384.0f);
    }
  }
  u32x4 x = {0, 0, 0, 0};
  const unsigned char* base = smem + (wave & 3) * 8192 + lane * 16;
  uint32_t off = 0;
  for (int it = 0; it < iters; ++it) {
    asm volatile("" : "+v"(off));                        // (keeps the reads inside the loop)
    u32x4 v[READS > 0 ? READS : 1];
#pragma unroll
    for (int r = 0; r < READS; ++r) v[r] = *reinterpret_cast<const u32x4*>(base + off + r * 1024);
#pragma unroll
    for (int a = 0; a < 8; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc[a], 0, 0, 0);
#pragma unroll
    for (int r = 0; r < READS; ++r) x ^= v[r];
  }
  float s = 0.f;
#pragma unroll
  for (int a = 0; a < 8; ++a) s += acc[a][0];
  if (s == 12345.f || x[0] == 0xdeadbeefu) sink[0] = x[1];
}
}  // namespace blr

extern "C" double blr_mfma_probe_flops(int iters) {
  const int cus = blr::device_cus() > 0 ? blr::device_cus() : 256;
  return (double)cus * 8.0 * (double)iters * 8.0 * (2.0 * 32 * 32 * 16);
}

extern "C" int blr_mfma_probe(int iters, int random, int lds_reads, void* dst, void* stream) {
  using namespace blr;
  if (iters <= 0 || !dst || (lds_reads != 0 && lds_reads != 6)) { set_error("mfma_probe: iters > 0, dst, lds_reads 0 or 6"); return BLR_ERR_BAD_ARG; }
  const int cus = device_cus() > 0 ? device_cus() : 256;
  hipStream_t st = (hipStream_t)stream;
  unsigned* sink = reinterpret_cast<unsigned*>(dst);
  if (random && lds_reads) hipLaunchKernelGGL((mfma_probe_kernel<true, 6>), dim3(cus), dim3(512), 0, st, sink, iters);
  else if (random) hipLaunchKernelGGL((mfma_probe_kernel<true, 0>), dim3(cus), dim3(512), 0, st, sink, iters);
  else if (lds_reads) hipLaunchKernelGGL((mfma_probe_kernel<false, 6>), dim3(cus), dim3(512), 0, st, sink, iters);
  else hipLaunchKernelGGL((mfma_probe_kernel<false, 0>), dim3(cus), dim3(512), 0, st, sink, iters);
  BLR_CHECK_LAUNCH("mfma_probe");
  return BLR_OK;
}

#ifdef BLR_TRACE
extern "C" int blr_debug_trace_gemm(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace_gemm), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

// BLAST at up to four token rows as two launches: stage 1, then mix + stage 2.
//
// A hand-over between workgroups inside one launch (tagged store, polls that may come too early, a reduction on
// either side) costs about 1.5 us per hop on this chip, and the single-launch decode kernels have two or three of them
// on their critical path.  The boundary between two kernels of one stream costs 1.0 us from the last wave of the
// first to the first wave of the second - and what crosses it is ordinary, cached memory.  So:
//   * pair_stage1_kernel: workgroup = one item (input block j, 128 ranks, k-slice) of  y = x V.  Any number of
//     workgroups, nothing to wait for, y leaves as T through plain stores (the reference rounds Y to its 16-bit type
//     as well: triton_funcs/blast_kernels.py:276);
//   * pair_slab_kernel: workgroup = (output block i, column chunk) with the whole rank in registers.  It asks for its
//     mix operands (y of every input block, S of block i: 64 - 128 KiB that sit in L2 after the first slab of a block
//     has fetched them), then for its slab of U, computes  z_i = sum_j S_ij * y_j  redundantly with the other slabs of
//     block i while U streams, multiplies and stores.  No partial outputs, no tags, no epoch, no spinning, no
//     residency requirement.
// Where stage 1 has long items and U is small (deep input blocks: 11008 -> 4096), launch 1 carries extra workgroups that only
// load the slabs of U, each on the XCD whose L2 its slab's workgroup of launch 2 will read from (see the launcher).
// The number of slab loads is a template parameter: the compiler then knows how many loads follow the mix operands
// and waits for exactly those (loads under runtime branches make it wait for everything in flight).
// The layouts of the bmm names are served at one row as well (measured 12.0 -> 9.6, 20.2 -> 16.6 and 17.1 -> 14.0 us on the
// three Llama-7B layers against the single-launch kernel): U as (b, q, r) by a variant of the slab kernel whose slab is a
// run of whole rows of U_i, and S as (r, i, j) by letting launch 1 rewrite it, eight ranks per workgroup, in the order the
// mix reads.
#include <map>
#include <mutex>
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
constexpr int DP_NT = 512;
constexpr int DP_UNR1 = 8;            // 16-byte loads of a stage-1 item per lane
constexpr int DP_AS = 8192;           // floats of staged activations (x slice of stage 1; z of a slab)
constexpr int dp_ks_max(int MT) { return MT <= 1 ? 4 : (MT <= 2 ? 2 : 1); }   // most k-slices of stage 1 (their y pieces sit in registers of the mix)
constexpr int DP_JJ = 4;              // input blocks a mix thread combines
constexpr uint32_t DP_OOB = 0x80000000u;
constexpr int ilog2k(int v) { return v <= 1 ? 0 : 1 + ilog2k(v >> 1); }
}  // namespace

#ifdef BLR_TRACE
__device__ unsigned long long g_trace4[1024 * 16];
#define TR4(i) do { if (threadIdx.x == 0 && blockIdx.x < 512) g_trace4[(TR4_BASE + blockIdx.x) * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR4(i) do {} while (0)
#endif

struct PairParams {
  const void* x; int64_t ldx;
  const void* V; const void* U; const void* S;
  const f16* u_scales; const f16* v_scales;      // quantized weights only
  void* out; int64_t ldo;
  void* y;                                       // [ks1][b][M][R] of T
  int M, b, bo, P, R, Q;
  int64_t s_si, s_sj, s_sr, o_bs, o_ns;
  int lpr1_log2, ks1, kc1, nb1, kpad1_log2, x_vec;
  FastDiv nch1, bdiv;
  int lpr2_log2, pfn, kld2_log2, octs_log2, jpg;
  FastDiv nch2;
  int xcd_order;
  const void* bias; int act, ep;                 // fused output stage: bias of T (indexed like a row of out) or null, blr_act
  int pre_split;                                 // workgroups that share the fetch of one slab (each takes pre_loads / pre_split loads)
  int items1, grid2, pre_loads, qr;              // launch 1: workgroups of stage 1; behind them, one per slab of launch 2 that fetches the
                                                 // slab's first pre_loads loads into the L2 of the XCD its slab workgroup will run on
  int perm_per;                                  // Monarch: z_i[r] = y[r / per][i per + r % per] (no S); 0 otherwise
  const void* s_rij; int s_chunks;               // S given as (r, i, j): stage 1 rewrites it as (j, i, r) into S, eight ranks per workgroup
};

__device__ __forceinline__ void lds_barrier2() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rbuf2(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// Totals over the row groups of a workgroup (see decode3_kernel): red is [m][row group][column], a row of nc columns padded
// to nc + nc / 8 floats so that the lanes of a column, which read different row groups, meet different banks; every lane of
// a column ends up with its total (the lanes of a column are neighbours inside a row of 16 lanes: DPP adds, no LDS trips).
// red holds MT * 512 * EPL * 9 / 8 floats.
template <int MT, int EPL>
__device__ __forceinline__ void pair_reduce(float (&acc)[MT][EPL], int lpr_log2, float* red, float (&tot)[MT]) {
  const int tid = threadIdx.x;
  const int cv = tid & ((1 << lpr_log2) - 1), rs = tid >> lpr_log2;
  const int nc_log2 = lpr_log2 + ilog2k(EPL), nrs_log2 = 9 - lpr_log2, sub_log2 = 9 - nc_log2;
  const int ld = (1 << nc_log2) + (1 << (nc_log2 - 3));
  lds_barrier2();                                    // earlier readers of red are done
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; e += 4)
      *reinterpret_cast<f32x4*>(&red[((m << nrs_log2) + rs) * ld + cv * EPL + e]) = f32x4{acc[m][e], acc[m][e + 1], acc[m][e + 2], acc[m][e + 3]};
  lds_barrier2();
  const int col = tid >> sub_log2, sub = tid & ((1 << sub_log2) - 1);
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    float v = 0.0f;
#pragma unroll
    for (int t = 0; t < EPL; ++t) v += red[((m << nrs_log2) + sub + (t << sub_log2)) * ld + col];
    if (sub_log2 >= 1) v = dpp_add<0xB1>(v);           // lanes 1 0 3 2
    if (sub_log2 >= 2) v = dpp_add<0x4E>(v);           // lanes 2 3 0 1
    if (sub_log2 >= 3) v = dpp_add<0x141>(v);          // the other quad of eight lanes (row_half_mirror)
    if (sub_log2 >= 4) v = dpp_add<0x140>(v);          // the other half of sixteen lanes (row_mirror)
    tot[m] = v;
  }
}

// Where a slab workgroup's loads of U start: byte offset of this lane's first load, the uniform step between loads, and what
// decides whether load u exists (rows of U along the rank: the row of the load lies inside the block; otherwise u < pfn).
struct SlabLoads { uint32_t uoff, ustep; int qrow0, rppq; };
template <int WB>
__device__ __forceinline__ SlabLoads slab_loads(const PairParams& p, uint32_t w, int tid, bool qr) {
  constexpr int EPL = 128 / WB;
  const uint32_t i2 = fd_div(w, p.nch2), nc2 = w - i2 * p.nch2.d;
  SlabLoads s;
  if (qr) {
    const int oct = tid & ((1 << p.octs_log2) - 1), jg = tid >> p.octs_log2;
    s.rppq = DP_NT >> p.octs_log2;
    s.qrow0 = (int)nc2 * p.pfn * s.rppq + jg;              // (pfn is the slab kernel's whole load count in this layout)
    s.uoff = (uint32_t)(((int)i2 * p.Q + s.qrow0) * p.R + oct * 8) * 2u;
    s.ustep = (uint32_t)DP_NT * 16u;
  } else {
    const int lpr2 = 1 << p.lpr2_log2, rpp2 = DP_NT >> p.lpr2_log2;
    const int cv2 = tid & (lpr2 - 1), rs2 = tid >> p.lpr2_log2;
    const int n2 = (int)nc2 * lpr2 * EPL + cv2 * EPL;
    s.rppq = 0; s.qrow0 = 0;
    s.uoff = (uint32_t)((((int)i2 * p.R + rs2) * p.Q + (n2 < p.Q ? n2 : 0))) * (uint32_t)WB / 8u;
    s.ustep = (uint32_t)rpp2 * (uint32_t)p.Q * (uint32_t)WB / 8u;
  }
  return s;
}

// ---- launch 1: y[ks][j][m][n] = sum_k x[m, j P + k] V_j[k, n] over one k-slice -------------------------------------------
template <typename T, int MT, int WB, bool ST>
__global__ __launch_bounds__(DP_NT) void pair_stage1_kernel(PairParams p) {
  constexpr int TR4_BASE = 0; (void)TR4_BASE;
  constexpr int EPL = 128 / WB;
  __shared__ __attribute__((aligned(16))) float a_s[4096];
  __shared__ __attribute__((aligned(16))) float red[MT * DP_NT * EPL * 9 / 8];
  const int tid = threadIdx.x;
  TR4(0);
  if (blockIdx.x >= (uint32_t)p.items1) {
    // Not a stage-1 item: this workgroup pulls the head of one slab of U into L2 while stage 1 leaves most of the memory system
    // idle.  It picks the slab whose workgroup of launch 2 will run on the same XCD (workgroup w runs on XCD w % 8, and the L2 is
    // per XCD): blocks of eight consecutive slab indices are permuted so that index and own index agree modulo 8.
    const uint32_t g8 = ((uint32_t)p.grid2 + 7u) & ~7u;
    const uint32_t q = blockIdx.x, tq = q - (uint32_t)p.items1;
    const uint32_t part = tq / g8, t = tq - part * g8;
    const uint32_t b2 = (t & ~7u) + (q & 7u);
    if (b2 >= (uint32_t)p.grid2) return;
    const int per_part = p.pre_loads / p.pre_split, u_lo = (int)part * per_part, u_hi = u_lo + per_part;
    const uint32_t w2 = p.xcd_order ? xcd_item(b2, (uint32_t)p.grid2) : b2;
    const SlabLoads sl = slab_loads<WB>(p, w2, tid, p.qr != 0);
    const __amdgpu_buffer_rsrc_t ub = rbuf2(p.U, (uint32_t)((int64_t)p.bo * p.R * p.Q * WB / 8));   // plain cached loads: the lines should stay
    for (int u0 = u_lo; u0 < u_hi; u0 += 8) {
      u32x4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const bool on = u0 + u < u_hi && (p.qr ? sl.qrow0 + (u0 + u) * sl.rppq < p.Q : u0 + u < p.pfn);
        v[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ub, on ? sl.uoff : DP_OOB, (uint32_t)(u0 + u) * sl.ustep, 0));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) asm volatile("" ::"v"(v[u]));
    }
    return;
  }
  const int M = p.M;
  const int lpr1 = 1 << p.lpr1_log2, rpp1 = DP_NT >> p.lpr1_log2;
  const int cv1 = tid & (lpr1 - 1), rs1 = tid >> p.lpr1_log2;
  const int kpad1 = 1 << p.kpad1_log2;
  const int nl1 = p.kc1 >> (9 - p.lpr1_log2);            // loads per lane that cover a slice
  const __amdgpu_buffer_rsrc_t vbuf = wbuf(p.V, (uint32_t)((int64_t)p.b * p.P * p.R * WB / 8));
  const __amdgpu_buffer_rsrc_t xbuf = rbuf2(p.x, (uint32_t)(((int64_t)(M - 1) * p.ldx + (int64_t)p.b * p.P) * 2));
  const uint32_t vstep = (uint32_t)rpp1 * (uint32_t)p.R * (uint32_t)WB / 8u;
  const uint32_t it = blockIdx.x;
  const uint32_t t1 = fd_div(it, p.nch1), nc1 = it - t1 * p.nch1.d;
  const uint32_t ks = fd_div(t1, p.bdiv), j = t1 - ks * p.bdiv.d;
  const int n0 = (int)nc1 * lpr1 * EPL;
  const int k0 = (int)ks * p.kc1, kc = min(p.kc1, p.P - k0);
  // S as (r, i, j): the first rank / 8 workgroups turn eight ranks each into 16-byte pieces of the (j, i, r) order the mix
  // of launch 2 reads.  Thread = (i, j); its loads go out first and its store follows the loads of V, so nothing waits.
  const __amdgpu_buffer_rsrc_t srbuf = rbuf2(p.s_rij ? p.s_rij : p.x, p.s_rij ? (uint32_t)p.b * p.bo * p.R * 2u : 2u);
  const bool s_on = ST && it < (uint32_t)p.s_chunks && tid < p.b * p.bo;
  uint32_t s16[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  if (s_on) {                                              // (a load instruction costs its turn in the memory pipeline even when every lane is out of bounds)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      s16[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(srbuf, (uint32_t)(((int)it * 8 + e) * p.b * p.bo + tid) * 2u, 0, 0);
  }
  // the activations next (loads come back in order); outside the slice the offset is out of bounds and reads as zero
  u32x4 xq;
  if (p.x_vec) {
    if (tid * 8 < (MT << p.kpad1_log2)) {
      const int m = (tid * 8) >> p.kpad1_log2, ka = (tid * 8) & (kpad1 - 1);
      const uint32_t xo = (m < M && ka < kc) ? (uint32_t)(m * (int)p.ldx + (int)j * p.P + k0 + ka) * 2u : DP_OOB;
      xq = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xbuf, xo, 0, 0));
    }
  }
  // the piece of V: rows past the slice (the last slice of a block may be short) meet a zero activation
  const int n = n0 + cv1 * EPL;
  const uint32_t voff = (uint32_t)((((int)j * p.P + k0 + rs1) * p.R + (n < p.R ? n : 0))) * (uint32_t)WB / 8u;
  u32x4 raw[DP_UNR1];
  auto load_batch = [&](int bi) {                          // loads bi * 8 .. of the slice, branched around in groups
    const int left = nl1 - bi * DP_UNR1;
    const uint32_t so = (uint32_t)(bi * DP_UNR1) * vstep;
#pragma unroll
    for (int u = 0; u < DP_UNR1; ++u) raw[u] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < 2; ++u) raw[u] = ldw16(vbuf, u < left ? voff : DP_OOB, so + (uint32_t)u * vstep);
    if (left > 2) {
#pragma unroll
      for (int u = 2; u < 4; ++u) raw[u] = ldw16(vbuf, u < left ? voff : DP_OOB, so + (uint32_t)u * vstep);
    }
    if (left > 4) {
#pragma unroll
      for (int u = 4; u < 8; ++u) raw[u] = ldw16(vbuf, u < left ? voff : DP_OOB, so + (uint32_t)u * vstep);
    }
  };
  load_batch(0);
  TR4(1);
  if (ST && s_on) {
    const int si = tid / p.b, sj = tid - si * p.b;       // S[r][i][j] -> S_t[j][i][r]
    const u32x4 pk = {s16[0] | (s16[1] << 16), s16[2] | (s16[3] << 16), s16[4] | (s16[5] << 16), s16[6] | (s16[7] << 16)};
    *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(const_cast<void*>(p.S)) + ((int64_t)(sj * p.bo + si) * p.R + (int64_t)it * 8) * 2) = pk;
  }
  if (p.x_vec) {
    if (tid * 8 < (MT << p.kpad1_log2)) {
      const typename TypeTraits<T>::vec8 v = __builtin_bit_cast(typename TypeTraits<T>::vec8, xq);
      float* dst = &a_s[tid * 8];
      *reinterpret_cast<f32x4*>(dst) = f32x4{TypeTraits<T>::to_f32(v[0]), TypeTraits<T>::to_f32(v[1]), TypeTraits<T>::to_f32(v[2]), TypeTraits<T>::to_f32(v[3])};
      *reinterpret_cast<f32x4*>(dst + 4) = f32x4{TypeTraits<T>::to_f32(v[4]), TypeTraits<T>::to_f32(v[5]), TypeTraits<T>::to_f32(v[6]), TypeTraits<T>::to_f32(v[7])};
    }
  } else {
    for (int idx = tid; idx < (MT << p.kpad1_log2); idx += DP_NT) {
      const int m = idx >> p.kpad1_log2, ka = idx & (kpad1 - 1);
      const uint32_t xo = (m < M && ka < kc) ? (uint32_t)(m * (int)p.ldx + (int)j * p.P + k0 + ka) * 2u : DP_OOB;
      a_s[idx] = TypeTraits<T>::to_f32(__builtin_bit_cast(T, (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(xbuf, xo, 0, 0)));
    }
  }
  lds_barrier2();
  float acc[MT][EPL];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
  for (int bi = 0; bi < p.nb1; ++bi) {                     // one batch unless a slice is deeper than eight passes
    const int left = nl1 - bi * DP_UNR1;
    auto fma_group = [&](int u0, int u1) {
      float av[MT][4];
#pragma unroll
      for (int u = u0; u < u1; ++u)
#pragma unroll
        for (int m = 0; m < MT; ++m) av[m][u - u0] = a_s[(m << p.kpad1_log2) + rs1 + (bi * DP_UNR1 + u) * rpp1];
#pragma unroll
      for (int u = u0; u < u1; ++u) {
        float wv[EPL];
        cvtw<T, WB>(raw[u], wv);                           // slots without a load hold zeros
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(av[m][u - u0], wv[e], acc[m][e]);
      }
    };
    fma_group(0, 2);
    if (left > 2) fma_group(2, 4);
    if (left > 4) fma_group(4, 8);
    if (bi + 1 < p.nb1) load_batch(bi + 1);
  }
  TR4(2);
  float tot[MT];
  pair_reduce<MT, EPL>(acc, p.lpr1_log2, red, tot);
  const int sub_log2 = 9 - (p.lpr1_log2 + ilog2k(EPL));
  const int col = n0 + (tid >> sub_log2);
  if ((tid & ((1 << sub_log2) - 1)) == 0 && col < p.R) {
    float vsc = 1.0f;                                      // per-rank scale of the codes of V
    if constexpr (WB != 16) vsc = (float)p.v_scales[(int)j * p.R + col];
    T* yp = reinterpret_cast<T*>(p.y);
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (m < M) yp[(((int)ks * p.b + (int)j) * M + m) * p.R + col] = TypeTraits<T>::from_f32(tot[m] * vsc);
  }
  TR4(3);
}

// ---- launch 2: z_i = sum_j S_ij * y_j, then out_i = z_i U_i over a register-resident slab ---------------------------------
//
// QR: U_i is (q, r) row-major (the bmm names).  A slab is then PF * rows-per-pass whole rows of U_i, one contiguous run of
// memory read in linear order; a lane meets the same eight ranks in every load (its z sits in registers), keeps one
// partial dot product per load and row, and the partials of a row are added up across its lanes: two DPP steps inside
// the quad, one pass through LDS for the rest.  Needs rank = 8 * 2^n, 128 <= rank <= 4096.
// JJ: input blocks a mix thread combines at most, 2 or 4 - a load costs its turn in the memory pipeline even with every lane
// out of bounds, so calls whose threads combine one or two blocks (rank 512 with 16 blocks) get a kernel without the other two
// (4096 -> 4096 at one row: 9.8 -> 9.7 us, with U as (b, q, r) 9.9 -> 9.4 us).
template <typename T, int MT, int WB, int PFG, bool QR, int JJ>
__global__ __launch_bounds__(DP_NT) void pair_slab_kernel(PairParams p) {
  constexpr int TR4_BASE = 512; (void)TR4_BASE;
  constexpr int EPL = 128 / WB;
  constexpr int PF = 8 * PFG;
  static_assert(!QR || WB == 16, "rows of U along the rank: two-byte weights only");
  constexpr int KSM = dp_ks_max(MT);                 // k-slices of stage 1 this instantiation can add up
  using V8 = typename TypeTraits<T>::vec8;
  __shared__ __attribute__((aligned(16))) float a_s[DP_AS];
  __shared__ __attribute__((aligned(16))) float red[MT * DP_NT * EPL * 9 / 8];
  const int tid = threadIdx.x;
  TR4(0);
  const int M = p.M, R = p.R;
  const uint32_t w = p.xcd_order ? xcd_item(blockIdx.x, gridDim.x) : blockIdx.x;
  const uint32_t i2 = fd_div(w, p.nch2), nc2 = w - i2 * p.nch2.d;
  const int lpr2 = 1 << p.lpr2_log2, rpp2 = DP_NT >> p.lpr2_log2;
  const int cv2 = tid & (lpr2 - 1), rs2 = tid >> p.lpr2_log2;
  const int n0_2 = (int)nc2 * lpr2 * EPL;
  const int n2 = n0_2 + cv2 * EPL;
  const int rppq = DP_NT >> p.octs_log2;               // QR: rows of U a load of the workgroup covers
  const int q0 = (int)nc2 * PF * rppq;                 // QR: first row of the slab

  // ---- mix operands of this thread: 8 ranks (one 16-byte piece) of y and S for up to DP_JJ input blocks ----
  const int oct = tid & ((1 << p.octs_log2) - 1), jg = tid >> p.octs_log2;
  const bool mix_on = oct * 8 < R;
  const __amdgpu_buffer_rsrc_t ybuf = rbuf2(p.y, (uint32_t)p.ks1 * p.b * M * R * 2u);
  const __amdgpu_buffer_rsrc_t sbuf = rbuf2(p.S ? p.S : p.x, p.S ? (uint32_t)p.b * p.bo * R * 2u : 2u);
  const int ib = p.bo > 1 ? (int)i2 : 0;               // (a single output block: every slab uses S of block 0, or none)
  u32x4 yq[MT][KSM][JJ];
  u32x4 sq[JJ];
  // Monarch: the "mix" is a gather - the eight ranks of this thread come from one input block (the period is a multiple
  // of eight), so group 0 fetches that one piece of y and the other groups contribute nothing
  const int pj = p.perm_per > 0 ? (oct * 8) / p.perm_per : 0;
  const int pr = p.perm_per > 0 ? (int)i2 * p.perm_per + (oct * 8 - pj * p.perm_per) : oct * 8;
#pragma unroll
  for (int jj = 0; jj < JJ; ++jj) {
    const int j = p.perm_per > 0 ? pj : jg * p.jpg + jj;
    const bool on = p.perm_per > 0 ? (mix_on && jj == 0 && jg == 0) : (mix_on && jj < p.jpg && j < p.b);
    sq[jj] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, (on && p.S) ? (uint32_t)(ib * (int)p.s_si + j * (int)p.s_sj + oct * 8) * 2u : DP_OOB, 0, 0));
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int ks = 0; ks < KSM; ++ks)
        if (ks < p.ks1 && m < M)
          yq[m][ks][jj] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ybuf, on ? (uint32_t)(((ks * p.b + j) * M + m) * R + pr) * 2u : DP_OOB, 0, 0));
  }
  // ---- the whole slab of U right behind, in straight-line code: the compiler counts exactly these PF loads ----
  const __amdgpu_buffer_rsrc_t ubuf = wbuf(p.U, (uint32_t)((int64_t)p.bo * R * p.Q * WB / 8));
  const SlabLoads sl = slab_loads<WB>(p, w, tid, QR);
  const uint32_t uoff = sl.uoff, ustep = sl.ustep;
  auto u_on = [&](int u) { return QR ? sl.qrow0 + u * sl.rppq < p.Q : u < p.pfn; };   // QR: rows past the block are not read
  // A wave that asks for more than the memory path of its compute unit takes at once is held at the load until there
  // is room, so only the first eight loads go out before the mix; the rest follow group by group, each behind the
  // products of the group before (whose data has landed by then: loads come back in order).
  u32x4 pf[PF];
#pragma unroll
  for (int u = 0; u < 8; ++u) pf[u] = ldw16(ubuf, u_on(u) ? uoff : DP_OOB, (uint32_t)u * ustep);
  TR4(1);

  // ---- mix: this thread's partial z over its input blocks, to LDS as [jg][m][r] (in `red`), then summed into a_s ----
  float* zp = red;
  const int rld = (8 << p.octs_log2);                   // ranks per row of zp (a power of two >= R)
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (m < M) {
      float z8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) z8[e] = 0.0f;
#pragma unroll
      for (int jj = 0; jj < JJ; ++jj) {
        if (jj < p.jpg) {
          float y8[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) y8[e] = 0.0f;
#pragma unroll
          for (int ks = 0; ks < KSM; ++ks) {
            if (ks < p.ks1) {
              const V8 yv = __builtin_bit_cast(V8, yq[m][ks][jj]);
#pragma unroll
              for (int e = 0; e < 8; ++e) y8[e] += TypeTraits<T>::to_f32(yv[e]);
            }
          }
          const V8 s8 = __builtin_bit_cast(V8, sq[jj]);
#pragma unroll
          for (int e = 0; e < 8; ++e) z8[e] = fmaf(p.S ? TypeTraits<T>::to_f32(s8[e]) : 1.0f, y8[e], z8[e]);
        }
      }
      float* dst = &zp[(jg * MT + m) * rld + oct * 8];
      *reinterpret_cast<f32x4*>(dst) = f32x4{z8[0], z8[1], z8[2], z8[3]};
      *reinterpret_cast<f32x4*>(dst + 4) = f32x4{z8[4], z8[5], z8[6], z8[7]};
    }
  }
  lds_barrier2();
  {
    const int njg = DP_NT >> p.octs_log2;               // groups of input blocks
    for (int idx = tid; idx < (MT << p.kld2_log2); idx += DP_NT) {
      const int m = idx >> p.kld2_log2, k = idx & ((1 << p.kld2_log2) - 1);
      float v = 0.0f;
      if (m < M && k < R)
        for (int g = 0; g < njg; ++g) v += zp[(g * MT + m) * rld + k];
      a_s[idx] = v;                                      // zero beyond the rank: the last pass over a slab may reach past it
    }
  }
  lds_barrier2();
  TR4(2);

  auto store_out = [&](int m, int gn, float total) {       // one element of out: scale of the codes, fused bias / activation
    float usc = 1.0f;
    if constexpr (WB != 16) usc = (float)p.u_scales[(int64_t)i2 * p.Q + gn];
    const int64_t oc = (int64_t)i2 * p.o_bs + (int64_t)gn * p.o_ns;
    T r = TypeTraits<T>::from_f32(total * usc);
    if (p.ep) {                                            // on the rounded result, as a separate elementwise kernel would see it
      float v = TypeTraits<T>::to_f32(r);
      if (p.bias) v += TypeTraits<T>::to_f32(reinterpret_cast<const T*>(p.bias)[oc]);
      r = TypeTraits<T>::from_f32(apply_act(v, p.act));
    }
    reinterpret_cast<T*>(p.out)[(int64_t)m * p.ldo + oc] = r;
  };
  if constexpr (QR) {
    // ---- rows of U along the rank: one partial dot product per load and token row ----
    float zr[MT][8];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(&a_s[(m << p.kld2_log2) + oct * 8]);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(&a_s[(m << p.kld2_log2) + oct * 8 + 4]);
#pragma unroll
      for (int e = 0; e < 4; ++e) { zr[m][e] = lo[e]; zr[m][4 + e] = hi[e]; }
    }
    float part[MT][PF];
#pragma unroll
    for (int g = 0; g < PFG; ++g) {
      if (g + 1 < PFG) {
#pragma unroll
        for (int v = 0; v < 8; ++v) { const int u = (g + 1) * 8 + v; pf[u] = ldw16(ubuf, u_on(u) ? uoff : DP_OOB, (uint32_t)u * ustep); }
      }
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const int u = g * 8 + v;
        float wv[8];
        cvtw<T, 16>(pf[u], wv);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          float s = 0.0f;
#pragma unroll
          for (int e = 0; e < 8; ++e) s = fmaf(zr[m][e], wv[e], s);
          part[m][u] = s;
        }
      }
    }
    TR4(3);
    // quad totals, then lane c of a quad keeps load 4 g + c: `red` holds [m][g][quad][c], written in thread order
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int g4 = 0; g4 < PF / 4; ++g4) {
        float keep = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float v = part[m][g4 * 4 + c];
          v = dpp_add<0xB1>(v);                            // lanes 1 0 3 2
          v = dpp_add<0x4E>(v);                            // lanes 2 3 0 1
          keep = (tid & 3) == c ? v : keep;
        }
        red[(m * (PF / 4) + g4) * DP_NT + tid] = keep;
      }
    lds_barrier2();
    // a group of threads adds the quads of four rows (loads 4 g .. 4 g + 3 of one row slot) as 16-byte pieces
    const int nv_log2 = p.octs_log2 - 2;                   // quads per row of U
    const int tpg_log2 = nv_log2 < 4 ? nv_log2 : 4, tpg = 1 << tpg_log2;
    const int k = tid & (tpg - 1);
    const int ngroups = (PF / 4) * rppq;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m >= M) break;
      for (int gi = tid >> tpg_log2; gi < ngroups; gi += DP_NT >> tpg_log2) {
        const int g4 = gi >> (9 - p.octs_log2), rw = gi & (rppq - 1);
        const float* src = &red[(m * (PF / 4) + g4) * DP_NT + ((rw << nv_log2) << 2)];
        f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int qd = k; qd < (1 << nv_log2); qd += tpg) s += *reinterpret_cast<const f32x4*>(src + qd * 4);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          float v = s[c];
          v = dpp_add<0xB1>(v);
          v = dpp_add<0x4E>(v);
          if (tpg_log2 >= 3) v = dpp_add<0x141>(v);        // the other quad of eight lanes (row_half_mirror)
          if (tpg_log2 >= 4) v = dpp_add<0x140>(v);        // the other half of sixteen lanes (row_mirror)
          s[c] = v;
        }
        if (k == 0) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int gn = q0 + (g4 * 4 + c) * rppq + rw;
            if (gn < p.Q) store_out(m, gn, s[c]);
          }
        }
      }
    }
    TR4(4);
    return;
  }
  // ---- products over the register-resident slab, eight loads at a time ----
  float acc[MT][EPL];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
  constexpr int GV = MT <= 2 ? 8 : 4;
#pragma unroll
  for (int g = 0; g < PFG; ++g) {
    if (g + 1 < PFG) {
#pragma unroll
      for (int v = 0; v < 8; ++v) { const int u = (g + 1) * 8 + v; pf[u] = ldw16(ubuf, u_on(u) ? uoff : DP_OOB, (uint32_t)u * ustep); }
    }
#pragma unroll
    for (int h = 0; h < 8 / GV; ++h) {
      const int u0 = g * 8 + h * GV;
      float av[MT][GV];
#pragma unroll
      for (int v = 0; v < GV; ++v)
#pragma unroll
        for (int m = 0; m < MT; ++m) av[m][v] = a_s[(m << p.kld2_log2) + ((rs2 + (u0 + v) * rpp2) & ((1 << p.kld2_log2) - 1))];
#pragma unroll
      for (int v = 0; v < GV; ++v) {
        float wv[EPL];
        cvtw<T, WB>(pf[u0 + v], wv);                     // slots without a load hold zeros
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(av[m][v], wv[e], acc[m][e]);
      }
    }
  }
  TR4(3);
  float tot[MT];
  pair_reduce<MT, EPL>(acc, p.lpr2_log2, red, tot);
  const int sub2_log2 = 9 - (p.lpr2_log2 + ilog2k(EPL));
  const int gn = n0_2 + (tid >> sub2_log2);
  if ((tid & ((1 << sub2_log2) - 1)) == 0 && gn < p.Q) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
      if (m < M) store_out(m, gn, tot[m]);
  }
  TR4(4);
}

// ---- host side --------------------------------------------------------------------------------------------------
namespace {
template <typename T, int MT, int WB, int JJ>
void* pair_slab_fn_jj(int pfg, bool qr) {
  if constexpr (WB == 16) {
    if (qr) {
      switch (pfg) {
        case 1: return (void*)pair_slab_kernel<T, MT, 16, 1, true, JJ>;
        case 2: return (void*)pair_slab_kernel<T, MT, 16, 2, true, JJ>;
        case 3: if constexpr (MT <= 2) return (void*)pair_slab_kernel<T, MT, 16, 3, true, JJ>; else return nullptr;
        case 4: if constexpr (MT <= 2) return (void*)pair_slab_kernel<T, MT, 16, 4, true, JJ>; else return nullptr;
        default: return nullptr;
      }
    }
  }
  if (qr) return nullptr;
  switch (pfg) {
    case 1: return (void*)pair_slab_kernel<T, MT, WB, 1, false, JJ>;
    case 2: return (void*)pair_slab_kernel<T, MT, WB, 2, false, JJ>;
    case 3: if constexpr (WB == 16) return (void*)pair_slab_kernel<T, MT, WB, 3, false, JJ>; else return nullptr;
    case 4: if constexpr (WB == 16) return (void*)pair_slab_kernel<T, MT, WB, 4, false, JJ>; else return nullptr;
    default: return nullptr;
  }
}
template <typename T, int MT, int WB>
void* pair_slab_fn(int pfg, bool qr, int jpg) {
  return jpg <= 2 ? pair_slab_fn_jj<T, MT, WB, 2>(pfg, qr) : pair_slab_fn_jj<T, MT, WB, DP_JJ>(pfg, qr);
}
// two-byte weights at 1, 2 and 4 token rows, int8 codes at 1 and 2, int4 codes at 1 (as decode3_kernel)
template <typename T>
bool pair_fns(int MT, int wbits, int pfg, bool qr, bool st, int jpg, void** f1, void** f2) {
  *f1 = *f2 = nullptr;
  if (wbits == 16) {
    if (MT == 1) { *f1 = st ? (void*)pair_stage1_kernel<T, 1, 16, true> : (void*)pair_stage1_kernel<T, 1, 16, false>; *f2 = pair_slab_fn<T, 1, 16>(pfg, qr, jpg); }
    else if (MT == 2) { *f1 = st ? (void*)pair_stage1_kernel<T, 2, 16, true> : (void*)pair_stage1_kernel<T, 2, 16, false>; *f2 = pair_slab_fn<T, 2, 16>(pfg, qr, jpg); }
    else { *f1 = st ? (void*)pair_stage1_kernel<T, 4, 16, true> : (void*)pair_stage1_kernel<T, 4, 16, false>; *f2 = pair_slab_fn<T, 4, 16>(pfg, qr, jpg); }
  } else if (wbits == 8) {
    if (MT == 1) { *f1 = (void*)pair_stage1_kernel<T, 1, 8, false>; *f2 = pair_slab_fn<T, 1, 8>(pfg, qr, jpg); }
    else if (MT == 2) { *f1 = (void*)pair_stage1_kernel<T, 2, 8, false>; *f2 = pair_slab_fn<T, 2, 8>(pfg, qr, jpg); }
  } else if (wbits == 4) {
    if (MT == 1) { *f1 = (void*)pair_stage1_kernel<T, 1, 4, false>; *f2 = pair_slab_fn<T, 1, 4>(pfg, qr, jpg); }
  }
  return *f1 && *f2;
}
}  // namespace

// Returns BLR_OK, a negative blr_status, or 1 when the call is not for these kernels.
int decode_pair_launch(const StreamBlastArgs& a, void* region, size_t region_bytes, hipStream_t st) {
  const int enabled = option_value(OPT_DECODE_PAIR, 1);
  if (!enabled) return 1;
  static const int dbg0 = env_i("BLR_D2_DEBUG", 0);
  auto decline = [&](int line) { if (dbg0) fprintf(stderr, "decode pair: not for this call (line %d)\n", line); return 1; };
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int P = a.in_f / a.b, Q = a.out_f / bo, R = a.r, b = a.b, M = a.M;
  if (M < 1 || M > 4) return decline(__LINE__);
  if (a.wbits == 8 && M > 2) return decline(__LINE__);              // codes at more rows: the matrix-core kernel
  if (a.wbits == 4 && M > 1) return decline(__LINE__);
  if (a.perm_per > 0 && (a.S || a.perm_per % 8 || bo != b || a.perm_per * b != R)) return decline(__LINE__);   // Monarch: whole 16-byte pieces of one input block
  const bool qr = a.u_layout == BLR_U_QR;           // U (b, q, r): two-byte weights with a power-of-two rank of at least 128
  if (qr && (a.wbits != 16 || R < 128 || (R & (R - 1)))) return decline(__LINE__);
  if (!qr && a.u_layout != BLR_U_RQ) return decline(__LINE__);
  if (b > 16 * DP_JJ || b >= 65536 || bo >= 65536 || R % 8 || R > 4096) return decline(__LINE__);
  if (a.wbits != 16 && (!a.u_scales || !a.v_scales)) return decline(__LINE__);
  // 32-bit offsets into every operand, and DP_OOB has to lie beyond each of them
  if ((int64_t)a.in_f * R * 2 >= (int64_t)DP_OOB || (int64_t)a.out_f * R * 2 >= (int64_t)DP_OOB || (int64_t)b * bo * R * 2 >= (int64_t)DP_OOB ||
      ((int64_t)(M - 1) * a.ldx + a.in_f) * 2 >= (int64_t)DP_OOB) return decline(__LINE__);
  const int MT = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
  const int WBITS = a.wbits, EPL = 128 / WBITS;

  PairParams p = {};
  p.x = a.x; p.ldx = a.ldx; p.V = a.V; p.U = a.U; p.S = a.S; p.out = a.out; p.ldo = a.ldo;
  p.u_scales = (const f16*)a.u_scales; p.v_scales = (const f16*)a.v_scales;
  p.M = M; p.b = b; p.bo = bo; p.P = P; p.R = R; p.Q = Q; p.perm_per = a.perm_per;
  p.o_bs = a.out_ns ? a.out_bs : Q; p.o_ns = a.out_ns ? a.out_ns : 1;
  if (a.s_layout == BLR_S_JIR) { p.s_sj = (int64_t)b * R; p.s_si = R; p.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { p.s_sr = (int64_t)b * b; p.s_si = b; p.s_sj = 1; }
  else { p.s_si = (int64_t)b * R; p.s_sj = R; p.s_sr = 1; }
  // S as (r, i, j) with two-byte weights: rewritten by launch 1 into the scratch region as (j, i, r).  (Codes come with S in
  // that order too; they stay on the single-launch kernel, which measured 0.3 - 0.5 us faster on them.)
  const bool s_turn = a.S && a.s_layout == BLR_S_RIJ && a.wbits == 16;
  if (s_turn) {
    if (b * bo > DP_NT) return decline(__LINE__);
    p.s_sj = (int64_t)bo * R; p.s_si = R; p.s_sr = 1;
  }
  if (a.S && !s_turn && (p.s_sr != 1 || !aligned(a.S, 16))) return decline(__LINE__);     // S in 16-byte pieces along the rank
  p.x_vec = aligned(a.x, 16) && a.ldx % 8 == 0 && P % 8 == 0;

  // ---- stage 1: 128-rank chunks, k split so that an item is at most eight loads per lane; any number of workgroups ----
  {
    int lpr = 16;
    const int vecs = (R + EPL - 1) / EPL;
    while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
    const int rpp = DP_NT / lpr;
    const int nch = (vecs + lpr - 1) / lpr;
    const int cus = device_cus() > 0 ? device_cus() : 256;
    const int ks_max = dp_ks_max(MT);
    int ks = 1;
    // Few, fat items: every k-slice is one more partial y that each slab has to fetch and add in its mix, which costs more
    // than the idle compute units of this short kernel (measured: two slices 9.0 / 14.6 us, four / three slices 9.35 / 15.6 us
    // on 4096 -> 4096 and 11008 -> 4096).  An item may take two batches of loads; slices are added only up to half the chip.
    while (ks < ks_max && cdiv(cdiv(P, ks), rpp) > 2 * DP_UNR1) ++ks;
    while (ks < ks_max && (int64_t)b * nch * ks < cus / 2 && cdiv(cdiv(P, ks + 1), rpp) >= 2) ++ks;
    int kc = (int)cdiv(P, ks);
    kc = (int)cdiv(kc, rpp) * rpp;
    ks = (int)cdiv(P, kc);
    const int nb = (int)cdiv(kc / rpp, DP_UNR1);
    int kpad = 1;
    while (kpad < nb * DP_UNR1 * rpp) kpad <<= 1;
    if (MT * kpad > 4096) return d2_bail(__LINE__);
    p.nb1 = nb;
    p.lpr1_log2 = ilog2(lpr); p.nch1 = fd_make((uint32_t)nch); p.bdiv = fd_make((uint32_t)b);
    p.ks1 = ks; p.kc1 = kc; p.kpad1_log2 = ilog2(kpad);
  }
  p.xcd_order = 1;
  { const void* eb = nullptr; int ea = 0; if (epilogue_pending(&eb, &ea)) { p.ep = 1; p.bias = eb; p.act = ea; } }
  const size_t ybytes = ((size_t)p.ks1 * b * M * R * 2 + 255) / 256 * 256;
  const size_t sbytes = s_turn ? (size_t)b * bo * R * 2 : 0;
  if (ybytes + sbytes > region_bytes) return d2_bail(__LINE__);
  p.y = region;
  if (s_turn) {
    p.s_rij = a.S; p.s_chunks = R / 8;
    p.S = reinterpret_cast<char*>(region) + ybytes;
    if (b * (int)p.nch1.d * p.ks1 < p.s_chunks) return decline(__LINE__);       // one chunk of S per workgroup of launch 1
  }

  // ---- mix + stage 2: a slab spans the whole rank; the narrowest column chunk that keeps it within the registers ----
  {
    const int cus = device_cus() > 0 ? device_cus() : 256;
    int best_lpr = 0, best_pfn = 0;
    double best = 1e30;
    if (qr) {                                          // whole rows of U_i: 8, 16, 24 or 32 loads per lane of 8 KiB per workgroup each
      const int rppq = DP_NT / (R / 8);
      for (int pfn = 8; pfn <= (MT <= 2 ? 32 : 16); pfn += 8) {
        const int nch = (int)cdiv(Q, pfn * rppq);
        const double est = (double)cdiv((int64_t)bo * nch, cus) * (0.6 + pfn * 8192.0 / 35e3);
        if (est < best) { best = est; best_lpr = 16; best_pfn = pfn; p.nch2 = fd_make((uint32_t)nch); }
      }
    }
    for (int lpr0 = 16; lpr0 >= 4 && !qr; lpr0 >>= 1) {
      if (lpr0 == 4 && WBITS == 16) continue;        // 64-byte pieces of a row only for codes
      int lpr = lpr0;
      const int vecs = (Q + EPL - 1) / EPL;
      while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
      const int rpp = DP_NT / lpr;
      const int pfn = (int)cdiv(R, rpp);
      if (pfn > (WBITS == 16 ? 32 : 16)) continue;
      const int nch = (vecs + lpr - 1) / lpr;
      const int64_t nslab = (int64_t)bo * nch;
      // time ~ bytes of the busiest compute unit: slabs per compute unit (rounded up) times the slab, plus narrow-piece penalty
      const double slab_bytes = (double)pfn * rpp * lpr * 16.0;
      const double est = (double)cdiv(nslab, cus) * (0.6 + slab_bytes / 35e3) + (lpr < 16 ? (lpr < 8 ? 0.4 : 0.15) : 0.0);
      if (est < best) { best = est; best_lpr = lpr; best_pfn = pfn; p.nch2 = fd_make((uint32_t)nch); }
    }
    if (!best_lpr) return d2_bail(__LINE__);
    p.lpr2_log2 = ilog2(best_lpr); p.pfn = best_pfn;
    int kld = 1;
    while (kld < best_pfn * (DP_NT / best_lpr) || kld < R) kld <<= 1;
    if (MT * kld > DP_AS) return d2_bail(__LINE__);
    p.kld2_log2 = ilog2(kld);
    int octs = 1;
    while (octs * 8 < R) octs <<= 1;
    if (octs > DP_NT) return d2_bail(__LINE__);
    p.octs_log2 = ilog2(octs);
    const int njg = DP_NT / octs;
    p.jpg = (int)cdiv(b, njg);
    if (p.jpg > DP_JJ) return d2_bail(__LINE__);
    if ((size_t)njg * MT * octs * 8 > (size_t)MT * DP_NT * EPL) return d2_bail(__LINE__);     // partial z fits the reduction buffer
  }
  {
    // Slabs near the register limit (a long stream per compute unit) are better served by the single-launch kernel, which
    // runs stage 1 under that stream: 16.3 against 17.5 us at 4096 -> 22016, rank 1024; below that the two launches win
    // (9.5 against 10.6 us at 4096 -> 4096, rank 512).  BLR_DECODE_PAIR=2 takes every call this path can serve.
    const double slab_bytes = (double)p.pfn * (DP_NT >> p.lpr2_log2) * (1 << p.lpr2_log2) * 16.0;
    if (enabled != 2 && !qr && slab_bytes > 192.0 * 1024.0 && a.S && a.perm_per == 0 && bo > 1) return decline(__LINE__);
  }
  const int pfg = (p.pfn + 7) / 8;
  void *f1 = nullptr, *f2 = nullptr;
  const bool have = a.dtype == BLR_F16 ? pair_fns<f16>(MT, WBITS, pfg, qr, s_turn, p.jpg, &f1, &f2) : pair_fns<bf16>(MT, WBITS, pfg, qr, s_turn, p.jpg, &f1, &f2);
  if (!have) return d2_bail(__LINE__);
  const int grid1 = b * (int)p.nch1.d * p.ks1, grid2 = bo * (int)p.nch2.d;
  // Launch 1 also warms the L2 with U where its own items are long enough to hide that and all of U fits: extra workgroups,
  // each on the XCD where its slab's workgroup of launch 2 will run, load whole slabs and drop the data.  A slab's loads are
  // 8 KiB per workgroup each and a compute unit draws about 35 GB/s: a fetch that outlasts stage 1 only delays launch 2, one
  // that shares compute units with a short stage 1 slows it down, and a fetch of part of a long stream of U gains nothing.
  // Measured, without / with: 11008 -> 4096 (88 KiB items, 8 MB of U) 15.0 -> 13.9 us, low rank on that shape 15.1 -> 14.0,
  // Monarch 15.8 -> 15.2, low rank 4096 -> 4096 (64 KiB items, four workgroups per slab) 12.4 -> 11.7 (one per slab: 12.8);
  // 4096 -> 4096 (32 KiB items) 9.2 -> 9.4 - 9.6; 4096 -> 22016 (45 MB of U) 16.6 -> 17.1 - 18.3.  Hence: items of at least
  // 60 KB, whole slabs of at most 16 loads, at most 12 MB of U and no more slabs than compute units; as many workgroups per
  // slab (1, 2 or 4) as keep one's share within three quarters of an item.
  p.items1 = grid1; p.grid2 = grid2; p.qr = qr ? 1 : 0;
  {
    const double item_bytes = (double)p.kc1 * (1 << p.lpr1_log2) * 16.0;
    const double u_bytes = (double)bo * R * Q * WBITS / 8.0;
    const int cus = device_cus() > 0 ? device_cus() : 256;
    const int pfn8 = (int)cdiv(p.pfn, 8) * 8;
    int pre = (item_bytes >= 60e3 && pfn8 <= 16 && u_bytes <= 12e6 && grid2 <= cus) ? pfn8 : 0;
    int split = 1;
    while (split < 4 && pre * 8192.0 / split > 0.75 * item_bytes && pre % (2 * split) == 0) split *= 2;
    p.pre_loads = pre; p.pre_split = split;
  }
  const int grid1_all = grid1 + (p.pre_loads > 0 ? (int)cdiv(grid2, 8) * 8 * p.pre_split : 0);
  static const int dbg = env_i("BLR_D2_DEBUG", 0);
  if (dbg) fprintf(stderr, "decode pair: M=%d b=%d bo=%d P=%d R=%d Q=%d wb=%d | stage 1: %d items (ks %d, kc %d) | slabs %d (lpr %d, pfn %d, octs %d, jpg %d)\n",
                   M, b, bo, P, R, Q, WBITS, grid1, p.ks1, p.kc1, grid2, 1 << p.lpr2_log2, p.pfn, 1 << p.octs_log2, p.jpg);
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(f1, dim3(grid1_all), dim3(DP_NT), args, 0, st);
  if (e == hipSuccess) e = hipLaunchKernel(f2, dim3(grid2), dim3(DP_NT), args, 0, st);
  if (e != hipSuccess) { set_error("decode pair: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  if (p.ep) epilogue_taken();
  return BLR_OK;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace4(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace4), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

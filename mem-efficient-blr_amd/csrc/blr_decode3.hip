// Two-stage decode kernel for up to four token rows: one 512-thread workgroup per compute unit.
//
// The call  x V -> mix with S -> U  is a short dependency chain over 10 - 55 MB of weights, and three things measured
// on the chip shape the kernel:
//   * a compute unit draws 30 - 38 GB/s from memory however many loads it has in flight, and its vector memory
//     path returns loads in the order they were issued, across its waves.  What bounds the call is therefore the
//     largest share of bytes any one compute unit fetches, and a small hand-over load issued behind a deep stream
//     of weight loads waits for that stream;
//   * a hand-over (one tagged store, one device-scope load that sees it) costs 0.4 us on an idle chip and about
//     1 us under a full stream - but a poll that comes too early costs another round trip, and every step of the
//     chain that is not memory (index arithmetic, reductions, barriers) runs at two waves per SIMD, where
//     500 instructions are a microsecond;
//   * a workgroup of 512 threads is a whole compute unit: placement is not left to the dispatcher, a slab of U
//     spans the full rank (8 waves x 32 loads x 16 bytes = 256 KiB of registers), and stage 2 needs no k split.
// So a workgroup has one role.  "Chain" workgroups ask for their stage-1 items (pieces of V: what heads the chain is
// requested first) and, with no slab queued in front of their polls, the first of them run the mix; "slab" workgroups
// ask for their whole slab of U at once, without pacing.  A slab workgroup places a
// speculative fetch of its slice of z in front of its last eight loads: if the chain has delivered by the time
// three quarters of the slab have landed, the products run under the rest of the stream.  Index arithmetic uses
// shifts and multiply-high by launch constants, reductions go through LDS once.
// Hand-overs are tagged pairs {fp32 bits, epoch} as in decode2_kernel (same workspace block, same epoch protocol).
#include <map>
#include <mutex>
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
constexpr int D3_NT = 512;
constexpr int d3_pf(int WB) { return WB == 16 ? 32 : 16; }   // 16-byte loads of a slab of U per lane: all of it stays in registers
                                      // (codes: half as many, their widened form needs the room)
constexpr int D3_PFB = 8;             // ... of which the last ones go out behind the speculative fetch of z
constexpr int D3_UNR1 = 8;            // 16-byte loads of a stage-1 item per lane and batch
constexpr int D3_ITEMS = 2;           // stage-1 items a workgroup asks for up front
constexpr int D3_AS = 8192;           // floats of staged activations: two stage-1 items, or the z slice of a slab
constexpr int D3_KS1_MAX = 4;         // most k-slices of stage 1 (a mix thread fetches them all at once)
constexpr int D3_TAIL = 8;            // loads per lane and batch beyond the register-resident part of a slab
constexpr uint32_t D3_OOB = 0x80000000u;   // buffer offset beyond any factor: the load returns zero and touches no memory
constexpr int ilog2c(int v) { return v <= 1 ? 0 : 1 + ilog2c(v >> 1); }
}  // namespace

#ifdef BLR_TRACE
__device__ unsigned long long g_trace3[1024 * 16];
#define TR3(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) g_trace3[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR3(i) do {} while (0)
#endif

struct Decode3Params {
  const void* x; int64_t ldx;
  const void* V; const void* U; const void* S;
  const f16* u_scales; const f16* v_scales;      // quantized weights only
  void* out; int64_t ldo;
  int u_nk, rpw, kl_log2;                        // U (bo, q, r): rows of U per wave, log2 of the 16-byte loads per row and lane
  int perm_per; int64_t o_bs, o_ns;              // Monarch permutation period; output strides of (block, column)
  int zrep;                                      // bo == 1: z is published in zrep copies so that the slabs do not all poll one address range
  int M, b, bo, P, R, Q;                         // b blocks of the input (stage 1), bo blocks of the output (stage 2)
  int64_t s_si, s_sj, s_sr;
  int lpr1_log2, ks1, kc1, nb1, kpad1_log2, items1, nchain;
  FastDiv nch1, bdiv;
  int lpr2_log2, ks2, kc2, items2, pfn, kpad2, kld2_log2, zspec;
  FastDiv nch2, bodiv;
  int itemsM, rch_log2;
  int x_vec, s_mode;                             // activations in 16-byte pieces; S: 0 = any strides, 1 = r contiguous, 2 = j contiguous
  unsigned spin_limit;
  int xcd_order;
  const void* bias; int act, ep;                 // fused output stage: bias of T (indexed like a row of out) or null, blr_act
  unsigned long long* ypart;           // [ks1][b][M][R] tagged
  unsigned long long* zt;              // [bo or zrep][M][R] tagged
  unsigned long long* opart;           // [ks2 - 1][bo][M][Q] tagged
  unsigned* epoch_word; unsigned* arrive_word; unsigned* err_word;
};

// Workgroup barrier for data exchanged through LDS.  __syncthreads() also waits for every global load and store of
// the wave (it is a fence): behind a tagged store that is the 0.5 - 0.8 us until the store is acknowledged, and behind
// a prefetch it is the whole prefetch.  Nothing here hands global data between the waves of a workgroup.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Totals over the row groups of a workgroup.  Every thread holds EPL columns of one row group; red is laid out
// [m][row group][column], a row of nc columns padded to nc + nc / 8 floats so that the lanes of a column, which read
// different row groups, meet different banks.  Thread (column = tid >> sub, lane of SUB = 512 / columns) adds EPL row
// groups, then the SUB lanes of a column - neighbours inside a row of 16 lanes - add up by DPP: every lane of a column
// ends up with its total.  red holds MT * 512 * EPL * 9 / 8 floats.
template <int MT, int EPL>
__device__ __forceinline__ void wg_reduce_lds(float (&acc)[MT][EPL], int lpr_log2, float* red, float (&tot)[MT]) {
  const int tid = threadIdx.x;
  const int cv = tid & ((1 << lpr_log2) - 1), rs = tid >> lpr_log2;
  const int nc_log2 = lpr_log2 + ilog2c(EPL), nrs_log2 = 9 - lpr_log2, sub_log2 = 9 - nc_log2;
  const int ld = (1 << nc_log2) + (1 << (nc_log2 - 3));
  lds_barrier();                                   // earlier readers of red are done
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; e += 4)
      *reinterpret_cast<f32x4*>(&red[((m << nrs_log2) + rs) * ld + cv * EPL + e]) = f32x4{acc[m][e], acc[m][e + 1], acc[m][e + 2], acc[m][e + 3]};
  lds_barrier();
  const int col = tid >> sub_log2, sub = tid & ((1 << sub_log2) - 1);
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    float v = 0.0f;
#pragma unroll
    for (int t = 0; t < EPL; ++t) v += red[((m << nrs_log2) + sub + (t << sub_log2)) * ld + col];
    if (sub_log2 >= 1) v = dpp_add<0xB1>(v);         // lanes 1 0 3 2
    if (sub_log2 >= 2) v = dpp_add<0x4E>(v);         // lanes 2 3 0 1
    if (sub_log2 >= 3) v = dpp_add<0x141>(v);        // the other quad of eight lanes (row_half_mirror)
    if (sub_log2 >= 4) v = dpp_add<0x140>(v);        // the other half of sixteen lanes (row_mirror)
    tot[m] = v;
  }
}

// 16-bit, 32-bit and 64-bit accesses through buffer descriptors with 32-bit byte offsets (no 64-bit address arithmetic
// per access; an offset outside the descriptor reads as zero).  aux 17 = device-coherent (sc0 sc1).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rbuf(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
template <typename T>
__device__ __forceinline__ T ldb16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(T, (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
}
__device__ __forceinline__ void st_tag_b(__amdgpu_buffer_rsrc_t r, uint32_t off, float v, unsigned epoch) {
  __builtin_amdgcn_raw_buffer_store_b64(u32x2{__float_as_uint(v), epoch}, r, off, 0, 17);
}
__device__ __forceinline__ u32x2 ld_tag_b(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 17));
}

template <typename T, int MT, int WB>
__global__ __launch_bounds__(D3_NT) void decode3_kernel(Decode3Params p) {
  constexpr int EPL = 128 / WB;                      // weights per 16-byte load
  constexpr int ZR = MT <= 2 ? 2 : 1;                // 16-byte fetches of tagged z per lane and token row (two ranks each)
  constexpr int D3_PF = d3_pf(WB), D3_PFA = D3_PF - D3_PFB;
  __shared__ __attribute__((aligned(16))) float a_s[D3_AS];
  __shared__ __attribute__((aligned(16))) float red[MT * D3_NT * EPL * 9 / 8];
  __shared__ __attribute__((aligned(16))) T s_s[16 * D3_NT];   // a mix item's block of S as (i, j, r)
  const int tid = threadIdx.x;
  const int w = blockIdx.x, G = gridDim.x;
  const int M = p.M;
  TR3(0);
  // The epoch of the previous call: a plain, cached load (the word was last written before this kernel began, and
  // hundreds of workgroups asking one address for a device-scope copy would queue up at a single memory channel).
  // The tag of this call is formed from it where it is first needed, so that nothing waits for the load up here.
  const unsigned epoch_prev = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rbuf(p.epoch_word, 4), 0, 0, 0);
  unsigned epoch = 0;
  auto check_in = [&]() {
    epoch = epoch_prev + 1u;
    if (epoch == 0u) epoch = 1u;
    if (tid == 0) {
      asm volatile("" ::"v"(epoch) : "memory");
      (void)__hip_atomic_fetch_add(&p.arrive_word[(w % D2_SHARDS) * 64], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  const __amdgpu_buffer_rsrc_t ybuf = rbuf(p.ypart, (uint32_t)p.ks1 * p.b * M * p.R * 8u);
  const __amdgpu_buffer_rsrc_t zbuf = rbuf(p.zt, (uint32_t)(p.zrep > 1 ? p.zrep : p.bo) * M * p.R * 8u);

  if (w >= p.items2) {
    // ======================================= chain role: stage 1, then the mix =======================================
    const int c = w - p.items2;
    const bool mixer = c < p.itemsM;
    const int lpr1 = 1 << p.lpr1_log2, rpp1 = D3_NT >> p.lpr1_log2;
    const int cv1 = tid & (lpr1 - 1), rs1 = tid >> p.lpr1_log2;
    const int kpad1 = 1 << p.kpad1_log2;
    const int nl1 = p.kc1 >> (9 - p.lpr1_log2);            // loads per lane that cover a slice (kc1 is a multiple of the rows per pass)
    const __amdgpu_buffer_rsrc_t vbuf = wbuf(p.V, (uint32_t)((int64_t)p.b * p.P * p.R * WB / 8));
    const __amdgpu_buffer_rsrc_t xbuf = rbuf(p.x, (uint32_t)(((int64_t)(M - 1) * p.ldx + (int64_t)p.b * p.P) * 2));
    const uint32_t vstep = (uint32_t)rpp1 * (uint32_t)p.R * (uint32_t)WB / 8u;
    // the S values of a mix thread's (i, r) depend on nothing, so they are asked for first of all; they stay as loaded
    // (anything done to them up here would wait for them up here)
    // (Every vector memory instruction of a wave occupies the address path of the compute unit for some 16 cycles,
    // whatever its width: sixteen 2-byte loads per thread would cost the eight waves of a mix workgroup most of a
    // microsecond at the head of the chain, so S comes in 16-byte pieces where its layout allows.)
    uint32_t sv[16];                                    // mode 0: S(i, j = u, r); mode 2: pairs of j in sv[0 .. 7]
    u32x4 sq[2];                                        // mode 1: two pieces of 8 ranks of the item's (i, j, r) block, on their way to LDS
    const __amdgpu_buffer_rsrc_t sbuf = rbuf(p.S ? p.S : p.x, p.S ? (uint32_t)p.b * p.bo * p.R * 2u : 2u);
    if (mixer && p.S) {
      const int RCHs = 1 << p.rch_log2;
      const int g = min(tid >> p.rch_log2, p.bo - 1);   // (replicas of a single output block all use S of block 0)
      const int r = min((c << p.rch_log2) + (tid & (RCHs - 1)), p.R - 1);
      if (p.s_mode == 1) {
        // piece t of the block: 8 ranks r8 = t % (RCH / 8), then j, then i
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int t = tid + h * D3_NT;
          const int r8 = t & ((RCHs >> 3) - 1), jj = (t >> (p.rch_log2 - 3)) & 15, ii = t >> (p.rch_log2 + 1);
          const int rr0 = (c << p.rch_log2) + r8 * 8;
          const bool on = jj < p.b && ii < p.bo && rr0 < p.R && (t >> (p.rch_log2 - 3)) < 16 * 16;
          sq[h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, on ? (uint32_t)(ii * (int)p.s_si + jj * (int)p.s_sj + rr0) * 2u : D3_OOB, 0, 0));
        }
      } else if (p.s_mode == 2) {
        const uint32_t s0 = (uint32_t)(g * (int)p.s_si + r * (int)p.s_sr) * 2u;
        const u32x4 lo = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, s0, 0, 0));
        const u32x4 hi = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, s0 + 16u, 0, 0));
#pragma unroll
        for (int u = 0; u < 4; ++u) { sv[u] = lo[u]; sv[4 + u] = hi[u]; }
      } else {
        const uint32_t s0 = (uint32_t)(g * (int)p.s_si + r * (int)p.s_sr) * 2u, sj = (uint32_t)p.s_sj * 2u;
#pragma unroll
        for (int u = 0; u < 16; ++u) sv[u] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(sbuf, s0 + (uint32_t)min(u, p.b - 1) * sj, 0, 0);
      }
    }
    // ---- the stage-1 items of this workgroup: activations first (loads come back in order), then the pieces of V ----
    // A vector memory instruction occupies the address path of the compute unit for some 16 cycles whether or not its
    // offsets are inside the buffer, so loads a workgroup does not need are branched around (in groups), not sent
    // out of bounds one by one; a load under a branch of its own would be waited for at once.
    int it_j[D3_ITEMS], it_ks[D3_ITEMS], it_n0[D3_ITEMS];
    bool it_ok[D3_ITEMS];
    T xr[D3_ITEMS][2];
    u32x4 xq[D3_ITEMS];                                  // x_vec: piece tid of the slice (8 activations), threads below MT * kpad1 / 8
    u32x4 raw[D3_ITEMS][D3_UNR1];
#pragma unroll
    for (int q = 0; q < D3_ITEMS; ++q) {
      const int it = c + q * p.nchain;
      it_ok[q] = it < p.items1;
      const uint32_t itc = it_ok[q] ? (uint32_t)it : 0u;
      const uint32_t t1 = fd_div(itc, p.nch1), nc1 = itc - t1 * p.nch1.d;
      const uint32_t ks = fd_div(t1, p.bdiv), j = t1 - ks * p.bdiv.d;
      it_j[q] = (int)j; it_ks[q] = (int)ks; it_n0[q] = (int)nc1 * lpr1 * EPL;
      const int k0 = (int)ks * p.kc1, kc = min(p.kc1, p.P - k0);
      // x: element (m, ka) of the slice; outside the slice the offset is out of bounds (zero)
      if (p.x_vec) {
        if (tid < 64 * ((MT * kpad1 / 8 + 63) / 64)) {    // whole waves: the others issue nothing
          const int m = (tid * 8) >> p.kpad1_log2, ka = (tid * 8) & (kpad1 - 1);
          const uint32_t xo = (it_ok[q] && m < M && ka < kc) ? (uint32_t)(m * (int)p.ldx + (int)j * p.P + k0 + ka) * 2u : D3_OOB;
          xq[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xbuf, xo, 0, 0));
        }
      } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int idx = tid + h * D3_NT;
          const int m = idx >> p.kpad1_log2, ka = idx & (kpad1 - 1);
          const uint32_t xo = (it_ok[q] && m < M && ka < kc) ? (uint32_t)(m * (int)p.ldx + (int)j * p.P + k0 + ka) * 2u : D3_OOB;
          xr[q][h] = ldb16<T>(xbuf, xo);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < D3_ITEMS; ++q) {
      const int n = it_n0[q] + cv1 * EPL;
      const int k0 = it_ks[q] * p.kc1;
      // rows past the slice (the last slice of a block may be short) belong to the next slice: they meet a zero activation
      const uint32_t voff = (uint32_t)(((it_j[q] * p.P + k0 + rs1) * p.R + (n < p.R ? n : 0))) * (uint32_t)WB / 8u;
#pragma unroll
      for (int u = 0; u < D3_UNR1; ++u) raw[q][u] = u32x4{0u, 0u, 0u, 0u};
      if (it_ok[q]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) raw[q][u] = ldw16(vbuf, u < nl1 ? voff : D3_OOB, (uint32_t)u * vstep);
        if (nl1 > 2) {
#pragma unroll
          for (int u = 2; u < 4; ++u) raw[q][u] = ldw16(vbuf, u < nl1 ? voff : D3_OOB, (uint32_t)u * vstep);
        }
        if (nl1 > 4) {
#pragma unroll
          for (int u = 4; u < 8; ++u) raw[q][u] = ldw16(vbuf, u < nl1 ? voff : D3_OOB, (uint32_t)u * vstep);
        }
      }
    }
    TR3(11);
#pragma unroll
    for (int q = 0; q < D3_ITEMS; ++q) {
      if (p.x_vec) {
        if (tid < 64 * ((MT * kpad1 / 8 + 63) / 64) && tid * 8 < (MT << p.kpad1_log2)) {
          const typename TypeTraits<T>::vec8 v = __builtin_bit_cast(typename TypeTraits<T>::vec8, xq[q]);
          float* dst = &a_s[q * (D3_AS / D3_ITEMS) + tid * 8];
          *reinterpret_cast<f32x4*>(dst) = f32x4{TypeTraits<T>::to_f32(v[0]), TypeTraits<T>::to_f32(v[1]), TypeTraits<T>::to_f32(v[2]), TypeTraits<T>::to_f32(v[3])};
          *reinterpret_cast<f32x4*>(dst + 4) = f32x4{TypeTraits<T>::to_f32(v[4]), TypeTraits<T>::to_f32(v[5]), TypeTraits<T>::to_f32(v[6]), TypeTraits<T>::to_f32(v[7])};
        }
      } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int idx = tid + h * D3_NT;
          if (idx < (MT << p.kpad1_log2)) a_s[q * (D3_AS / D3_ITEMS) + idx] = TypeTraits<T>::to_f32(xr[q][h]);
        }
      }
    }
    if (mixer && p.S && p.s_mode == 1) {                 // the item's block of S to LDS as (i, j, r) of T, behind the activations
#pragma unroll
      for (int h = 0; h < 2; ++h) *reinterpret_cast<u32x4*>(&s_s[(tid + h * D3_NT) * 8]) = sq[h];
    }
    check_in();
    lds_barrier();
    TR3(13);
#pragma unroll
    for (int q = 0; q < D3_ITEMS; ++q) {
      if (!it_ok[q]) continue;                           // uniform over the workgroup
      const float* as = a_s + q * (D3_AS / D3_ITEMS);
      float acc[MT][EPL];
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
      auto fma_group = [&](int u0, int u1) {
        float av[MT][4];
#pragma unroll
        for (int u = u0; u < u1; ++u)
#pragma unroll
          for (int m = 0; m < MT; ++m) av[m][u - u0] = as[(m << p.kpad1_log2) + rs1 + u * rpp1];
#pragma unroll
        for (int u = u0; u < u1; ++u) {
          float wv[EPL];
          cvtw<T, WB>(raw[q][u], wv);                      // slots without a load hold zeros
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(av[m][u - u0], wv[e], acc[m][e]);
        }
      };
      fma_group(0, 2);
      if (nl1 > 2) fma_group(2, 4);
      if (nl1 > 4) fma_group(4, 8);
      if (q == 0) TR3(1);
      float tot[MT];
      wg_reduce_lds<MT, EPL>(acc, p.lpr1_log2, red, tot);
      const int sub_log2 = 9 - (p.lpr1_log2 + ilog2c(EPL));
      const int col = it_n0[q] + (tid >> sub_log2);
      if ((tid & ((1 << sub_log2) - 1)) == 0 && col < p.R) {
        float vsc = 1.0f;                                  // per-rank scale of the codes of V
        if constexpr (WB != 16) vsc = (float)p.v_scales[it_j[q] * p.R + col];
#pragma unroll
        for (int m = 0; m < MT; ++m)
          if (m < M) st_tag_b(ybuf, (uint32_t)(((it_ks[q] * p.b + it_j[q]) * M + m) * p.R + col) * 8u, tot[m] * vsc, epoch);
      }
    }
    TR3(2);
    // The call's epoch is closed by the last chain workgroup, as soon as it has nothing left to do (every workgroup checks in
    // before its first wait, so all of them have read the previous epoch by the time the count is complete) - at the end of a
    // slab workgroup the round trip of that count was the last thing the launch waited for.
    const bool closer = c == p.nchain - 1;
    if (!mixer) {
      if (closer) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
      return;
    }

    // ---- mix: z[i][m][r] = sum_j S(i, j, r) * sum_ks y[ks][j][m][r] for RCH values of r, every i ------------------
    // Thread (g, rr): first g is the input block j whose y it fetches, then the output block i it emits.
    lds_barrier();                                     // the stage-1 use of a_s is over
    TR3(8);
    const int RCH = 1 << p.rch_log2;
    const int g = tid >> p.rch_log2, rr = tid & (RCH - 1);
    const int r = (c << p.rch_log2) + rr;
    // Monarch: the "mix" is a permutation - z[l][r] is the single value y[r / per][l * per + r % per]
    const bool perm = p.perm_per > 0;
    int yj = g, yr = r;
    if (perm) { yj = r / p.perm_per; yr = g * p.perm_per + (r - yj * p.perm_per); }
    const bool live = (perm ? g < p.bo : g < p.b) && r < p.R;          // fetches y of input block yj
    const bool live_o = g < (p.zrep > 1 ? p.zrep : p.bo) && r < p.R;   // emits z of output block (or replica) g
    float ysum[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) ysum[m] = 0.0f;
    if (live) {
      u32x2 yv[D3_KS1_MAX][MT];
      const uint32_t y0 = (uint32_t)((yj * M) * p.R + yr) * 8u, yks = (uint32_t)(p.b * M * p.R) * 8u, ym = (uint32_t)p.R * 8u;
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int ks = 0; ks < D3_KS1_MAX; ++ks) {
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            if (ks < p.ks1 && m < M) {
              yv[ks][m] = ld_tag_b(ybuf, y0 + (uint32_t)ks * yks + (uint32_t)m * ym);
              ok = ok && yv[ks][m][1] == epoch;
            } else {
              yv[ks][m] = u32x2{0u, 0u};
            }
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
#pragma unroll
      for (int ks = 0; ks < D3_KS1_MAX; ++ks)
#pragma unroll
        for (int m = 0; m < MT; ++m) ysum[m] += __uint_as_float(yv[ks][m][0]);
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) a_s[m * D3_NT + tid] = ysum[m];     // [m][j][rr]
    lds_barrier();
    if (live_o) {
      float sf[16];
      if (!p.S) {
#pragma unroll
        for (int u = 0; u < 16; ++u) sf[u] = 1.0f;
      } else if (p.s_mode == 1) {
#pragma unroll
        for (int u = 0; u < 16; ++u) sf[u] = TypeTraits<T>::to_f32(s_s[((min(g, p.bo - 1) * 16 + u) << p.rch_log2) + rr]);
      } else {
#pragma unroll
        for (int u = 0; u < 16; ++u) asm volatile("" : "+v"(sv[u]));   // (keeps their widening - and the wait for them - down here)
#pragma unroll
        for (int u = 0; u < 16; ++u)
          sf[u] = TypeTraits<T>::to_f32(__builtin_bit_cast(T, (uint16_t)(p.s_mode == 2 ? sv[u >> 1] >> (16 * (u & 1)) : sv[u])));
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if (m < M) {
          float z = perm ? ysum[m] : 0.0f;
#pragma unroll
          for (int u = 0; u < 16; ++u)
            z = fmaf((u < p.b && !perm) ? sf[u] : 0.0f, a_s[m * D3_NT + min(u, p.b - 1) * RCH + rr], z);
          for (int j = 16; j < p.b && !perm; ++j)
            z = fmaf(p.S ? TypeTraits<T>::to_f32(ldb16<T>(sbuf, (uint32_t)(min(g, p.bo - 1) * (int)p.s_si + j * (int)p.s_sj + r * (int)p.s_sr) * 2u)) : 1.0f, a_s[m * D3_NT + j * RCH + rr], z);
          st_tag_b(zbuf, (uint32_t)((g * M + m) * p.R + r) * 8u, z, epoch);
        }
      }
    }
    TR3(9);
    if (closer) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
    return;
  }

  // ============================================== slab role ===========================================================
  // The whole slab of U is asked for at once.  Slots 0 .. PF - 9 hold the first pfn - 8 loads, the last eight slots the
  // last eight loads; groups of eight slots without a load are branched around, a single slot without one gets an
  // offset outside the buffer.  The speculative fetch of this slab's slice of z sits in front of the last group.
  const uint32_t ws2 = p.xcd_order ? xcd_item((uint32_t)w, (uint32_t)p.items2) : (uint32_t)w;   // slab of this workgroup
  const uint32_t t2 = fd_div(ws2, p.nch2), nc2 = ws2 - t2 * p.nch2.d;
  const uint32_t ksi2 = fd_div(t2, p.bodiv), i2 = t2 - ksi2 * p.bodiv.d;
  const int lpr2 = 1 << p.lpr2_log2, rpp2 = D3_NT >> p.lpr2_log2;
  const int cv2 = tid & (lpr2 - 1), rs2 = tid >> p.lpr2_log2;
  const int zi = p.zrep > 1 ? (int)(nc2 & (uint32_t)(p.zrep - 1)) : (int)i2;     // which published copy of z this slab reads
  const int k0_2 = (int)ksi2 * p.kc2;
  const int kcur2 = min(p.kc2, p.R - k0_2);
  const int n0_2 = (int)nc2 * lpr2 * EPL;
  const int n2 = n0_2 + cv2 * EPL;
  const __amdgpu_buffer_rsrc_t ubuf = wbuf(p.U, (uint32_t)((int64_t)p.bo * p.R * p.Q * WB / 8));
  const uint32_t uoff = (uint32_t)((((int)i2 * p.R + k0_2 + rs2) * p.Q + (n2 < p.Q ? n2 : 0))) * (uint32_t)WB / 8u;
  const uint32_t ustep = (uint32_t)rpp2 * (uint32_t)p.Q * (uint32_t)WB / 8u;
  const int nbq = p.pfn < D3_PFB ? p.pfn : D3_PFB, naq = p.pfn - nbq;    // loads in the last group, loads before it
  const int pairs = kcur2 >> 1;
  const uint32_t z0 = (uint32_t)((zi * M) * p.R + k0_2 + 2 * tid) * 8u;
  auto z_fetch = [&](u32x4 (&zv)[MT][ZR]) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int h = 0; h < ZR; ++h) {
        if (m < M && h * D3_NT < pairs) {
          const int kp = tid + h * D3_NT;
          zv[m][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(zbuf, kp < pairs ? z0 + (uint32_t)(m * p.R + 2 * h * D3_NT) * 8u : D3_OOB, 0, 17));
        }
      }
  };
  u32x4 pf[D3_PF];
  u32x4 zv[MT][ZR];
#pragma unroll
  for (int g8 = 0; g8 < D3_PFA / 8; ++g8) {
    if (g8 * 8 < naq) {
#pragma unroll
      for (int v = 0; v < 8; ++v) { const int u = g8 * 8 + v; pf[u] = ldw16(ubuf, u < naq ? uoff : D3_OOB, (uint32_t)u * ustep); }
    }
  }
  if (p.zspec) z_fetch(zv);
#pragma unroll
  for (int u = 0; u < D3_PFB; ++u) pf[D3_PFA + u] = ldw16(ubuf, u < nbq ? uoff : D3_OOB, (uint32_t)(naq + u) * ustep);
  TR3(12);
  check_in();

  // ---- this slab's slice of z into LDS: the speculative fetch if it caught this call's values, else polled ----
  const int kld2 = 1 << p.kld2_log2;
  {
    bool ok = p.zspec != 0;
    unsigned spins = 0;
    while (true) {
      if (ok) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int h = 0; h < ZR; ++h)
            if (m < M && tid + h * D3_NT < pairs) ok = ok && zv[m][h][1] == epoch && zv[m][h][3] == epoch;
      }
      if (__syncthreads_and(ok)) break;
      if (++spins > p.spin_limit) {
        if (tid == 0) __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      z_fetch(zv);
      ok = true;
    }
    TR3(4);
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int h = 0; h < ZR; ++h) {
        const int kp = tid + h * D3_NT;
        if (m < M && kp < pairs)
          *reinterpret_cast<float2*>(&a_s[(m << p.kld2_log2) + 2 * kp]) = float2{__uint_as_float(zv[m][h][0]), __uint_as_float(zv[m][h][2])};
      }
    // zero what the products touch beyond the slice: k in [kcur2, kpad2) (the last slice of a block may be short)
    if (p.kpad2 > kcur2) {
      for (int idx = tid; idx < MT * kld2; idx += D3_NT) {
        const int k = idx & (kld2 - 1);
        if (k >= kcur2 && k < p.kpad2) a_s[idx] = 0.0f;
      }
    }
    lds_barrier();
  }

  // ---- out[m, i Q + n] = sum_k z[m][k] U_i[k, n] over the register-resident slab, a group of loads at a time ----
  float acc[MT][EPL];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
  constexpr int GV = MT <= 2 ? 8 : 4;                  // slots whose activations are read from LDS together
#pragma unroll
  for (int g8 = 0; g8 < D3_PF / GV; ++g8) {
    const bool last = g8 * GV >= D3_PFA;
    if (last ? (g8 * GV - D3_PFA) < nbq : g8 * GV < naq) {
      float av[MT][GV];
#pragma unroll
      for (int v = 0; v < GV; ++v) {
        const int s = g8 * GV + v;
        const int u = last ? naq + (s - D3_PFA) : s;       // rows of a slot without a load lie in the zeroed part or meet zero weights
#pragma unroll
        for (int m = 0; m < MT; ++m) av[m][v] = (last && (s - D3_PFA) >= nbq) ? 0.0f : a_s[(m << p.kld2_log2) + ((rs2 + u * rpp2) & (kld2 - 1))];
      }
#pragma unroll
      for (int v = 0; v < GV; ++v) {
        float wv[EPL];
        cvtw<T, WB>(pf[g8 * GV + v], wv);                // slots without a load hold zeros
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(av[m][v], wv[e], acc[m][e]);
      }
    }
  }
  TR3(5);
  float tot[MT];
  wg_reduce_lds<MT, EPL>(acc, p.lpr2_log2, red, tot);
  TR3(6);
  const int sub2_log2 = 9 - (p.lpr2_log2 + ilog2c(EPL));
  const int gn = n0_2 + (tid >> sub2_log2);
  if ((tid & ((1 << sub2_log2) - 1)) == 0 && gn < p.Q) {
    if (ksi2 != 0) {                                  // a producer of partial sums
#pragma unroll
      for (int m = 0; m < MT; ++m)
        if (m < M) st_tag(&p.opart[(((int64_t)(ksi2 - 1) * p.bo + i2) * M + m) * p.Q + gn], tot[m], epoch);
    } else {                                          // the slab of k-slice 0 adds the others in order
      float usc = 1.0f;
      if constexpr (WB != 16) usc = (float)p.u_scales[(int64_t)i2 * p.Q + gn];   // per-output scale of the codes of U
      T* outp = reinterpret_cast<T*>(p.out);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if (m < M) {
          float v = tot[m];
          for (int ks = 1; ks < p.ks2; ++ks) {
            const unsigned long long* src = &p.opart[(((int64_t)(ks - 1) * p.bo + i2) * M + m) * p.Q + gn];
            unsigned long long pv;
            unsigned spins = 0;
            while (true) {
              pv = ld_tag(src);
              if ((unsigned)(pv >> 32) == epoch) break;
              if (++spins > p.spin_limit) {
                __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
              }
            }
            v += __uint_as_float((unsigned)pv);
          }
          {
            const int64_t oc = (int64_t)i2 * p.o_bs + (int64_t)gn * p.o_ns;
            T r = TypeTraits<T>::from_f32(v * usc);
            if (p.ep) {                                  // on the rounded result, as a separate elementwise kernel would see it
              float e = TypeTraits<T>::to_f32(r);
              if (p.bias) e += TypeTraits<T>::to_f32(reinterpret_cast<const T*>(p.bias)[oc]);
              r = TypeTraits<T>::from_f32(apply_act(e, p.act));
            }
            outp[(int64_t)m * p.ldo + oc] = r;
          }
        }
      }
    }
  }
  TR3(7);
}

// ---- host side --------------------------------------------------------------------------------------------------
namespace {
// the instantiations that exist: two-byte weights at 1, 2 and 4 token rows, int8 codes at 1 and 2, int4 codes at 1
// (wider accumulators do not fit next to a register-resident slab; those calls take the matrix-core kernel)
template <typename T>
void* d3_kernel(int MT, int wbits) {
  if (wbits == 8) return MT == 1 ? (void*)decode3_kernel<T, 1, 8> : MT == 2 ? (void*)decode3_kernel<T, 2, 8> : nullptr;
  if (wbits == 4) return MT == 1 ? (void*)decode3_kernel<T, 1, 4> : nullptr;
  return MT == 1 ? (void*)decode3_kernel<T, 1, 16> : MT == 2 ? (void*)decode3_kernel<T, 2, 16> : (void*)decode3_kernel<T, 4, 16>;
}
// microseconds a compute unit needs to have `bytes` of a cold stream in its registers: start-up plus 35 GB/s (what one
// compute unit draws with its queues full; measured 30 - 38 GB/s)
double d3_stream_us(double bytes) { return 0.6 + bytes / 35e3; }
}  // namespace

int decode3_blast_launch(const StreamBlastArgs& a, void* region, unsigned* epoch_word, unsigned* arrive_word,
                         unsigned* err_word, hipStream_t st) {
  const int enabled = option_value(OPT_DECODE3, 1);
  if (!enabled) return 1;
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int P = a.in_f / a.b, Q = a.out_f / bo, R = a.r, b = a.b, M = a.M;
  if (M < 1 || M > 4) return 1;
  if (a.wbits == 8 && M > 2) return 1;              // codes at more rows: the matrix-core kernel
  if (a.wbits == 4 && M > 1) return 1;
  if (a.u_layout == BLR_U_QR) return 1;             // U (b, q, r): decode2_kernel
  if (b >= 65536 || bo >= 65536 || R >= (1 << 20)) return 1;
  const int MT = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
  const int WBITS = a.wbits, EPL = 128 / WBITS;
  void* fn = a.dtype == BLR_F16 ? d3_kernel<f16>(MT, WBITS) : d3_kernel<bf16>(MT, WBITS);
  if (!fn) return 1;
  static std::mutex mu;
  static std::map<void*, int> occ_cache;
  int occ = 0;
  {
    std::lock_guard<std::mutex> lk(mu);
    auto it = occ_cache.find(fn);
    if (it != occ_cache.end()) occ = it->second;
    else {
      hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, D3_NT, 0);
      if (e != hipSuccess || occ < 1) { (void)hipGetLastError(); set_error("decode3: occupancy query failed"); return BLR_ERR_LAUNCH; }
      occ_cache[fn] = occ;
    }
  }
  const int resident = device_cus() > 0 ? device_cus() : 256;     // one workgroup per compute unit

  Decode3Params p = {};
  p.x = a.x; p.ldx = a.ldx; p.V = a.V; p.U = a.U; p.S = a.S; p.out = a.out; p.ldo = a.ldo;
  p.u_scales = (const f16*)a.u_scales; p.v_scales = (const f16*)a.v_scales;
  p.M = M; p.b = b; p.bo = bo; p.P = P; p.R = R; p.Q = Q;
  p.perm_per = a.perm_per; p.o_bs = a.out_ns ? a.out_bs : Q; p.o_ns = a.out_ns ? a.out_ns : 1;
  if (a.s_layout == BLR_S_JIR) { p.s_sj = (int64_t)b * R; p.s_si = R; p.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { p.s_sr = (int64_t)b * b; p.s_si = b; p.s_sj = 1; }
  else { p.s_si = (int64_t)b * R; p.s_sj = R; p.s_sr = 1; }
  p.spin_limit = spin_limit_now();
  p.xcd_order = 1;
  { const void* eb = nullptr; int ea = 0; if (epilogue_pending(&eb, &ea)) { p.ep = 1; p.bias = eb; p.act = ea; } }
  p.x_vec = aligned(a.x, 16) && a.ldx % 8 == 0 && P % 8 == 0;
  p.s_mode = 0;
  if (a.S && aligned(a.S, 16) && b <= 16 && R % 8 == 0) {
    if (p.s_sr == 1 && p.s_si % 8 == 0 && p.s_sj % 8 == 0) p.s_mode = 1;
    else if (p.s_sj == 1 && b == 16 && p.s_si % 8 == 0 && p.s_sr % 8 == 0) p.s_mode = 2;
  }

  // ---- the mix: 512 threads = (block, rank) pairs ---------------------------------------------------------------
  p.zrep = bo == 1 ? 16 : 1;
  int bp2 = 1;
  while (bp2 < b || bp2 < bo || bp2 < p.zrep) bp2 <<= 1;
  if (bp2 > D3_NT) return d2_bail(__LINE__);
  const int rch = D3_NT / bp2;
  p.rch_log2 = ilog2(rch);
  p.itemsM = (R + rch - 1) / rch;
  if (MT * D3_NT > D3_AS) return d2_bail(__LINE__);
  const int min_chain = p.itemsM > 16 ? p.itemsM : 16;
  if (min_chain >= resident) return d2_bail(__LINE__);

  // ---- stage 1 for a given number of slab and chain workgroups; false when it does not fit ----------------------
  struct S1 { int lpr, nch, ks, kc, nb, kpad, items, nchain; double t_chain; };
  auto plan1 = [&](int nslab, double slab_bytes, S1& s) -> bool {
    const int navail = resident - nslab;
    int lpr = 16;
    const int vecs = (R + EPL - 1) / EPL;
    while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
    const int rpp = D3_NT / lpr;
    const int nch = (vecs + lpr - 1) / lpr;
    const int base = b * nch;
    auto loads_of = [&](int ks) { return (int)cdiv(cdiv(P, ks), rpp); };
    bool have = false;
    double best = 1e30;
    {
      const int takers = D3_ITEMS * navail;
      for (int ks = 1; ks <= D3_KS1_MAX; ++ks) {
        int kc = (int)cdiv(P, ks);
        kc = (int)cdiv(kc, rpp) * rpp;
        if ((int)cdiv(P, kc) != ks) continue;
        const int loads = (int)cdiv(kc, rpp);
        const int nb = 1;
        if (loads > D3_UNR1) continue;                   // an item is one batch of loads
        const int kpad = D3_UNR1 * rpp;
        if (MT * kpad > 2 * D3_NT) continue;             // two activations per thread are staged
        const int items = base * ks;
        if (items > takers) continue;
        int nchain = items < navail ? items : navail;
        if (nchain < p.itemsM) nchain = p.itemsM;
        if (nchain > navail) continue;
        const double item_bytes = (double)kc * lpr * 16.0;
        const double t_chain = d3_stream_us(item_bytes * (double)cdiv(items, nchain)) + 0.3 * (double)cdiv(items, nchain);
        const double t_slab = d3_stream_us(slab_bytes);
        const double est = t_chain + 2.2 > t_slab ? t_chain + 2.2 : t_slab;     // chain: + two hand-overs and the mix
        if (est < best) {
          best = est; have = true;
          s = {lpr, nch, ks, kc, nb, kpad, items, nchain, t_chain};
        }
      }
    }
    return have;
  };

  S1 s1 = {};
  {
    // stage 2 on U (bo, r, q): the cut (lanes per row, k-slices) with the smallest estimated time
    double best = 1e30;
    bool found = false;
    for (int lpr0 = 16; lpr0 >= 4; lpr0 >>= 1) {
      if (lpr0 == 4 && WBITS == 16) continue;        // 64-byte pieces of a row only for codes
      int lpr = lpr0;
      const int vecs = (Q + EPL - 1) / EPL;
      while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
      const int rpp = D3_NT / lpr;
      const int nch = (vecs + lpr - 1) / lpr;
      for (int ks0 = 1; ks0 <= 4; ++ks0) {
        int kc = (int)cdiv(R, ks0);
        kc = (int)cdiv(kc, rpp) * rpp;
        const int ks = (int)cdiv(R, kc);
        if (ks != ks0) continue;
        const int pfn = kc / rpp;
        if (pfn > d3_pf(WBITS)) continue;                // the whole slab stays in registers
        const int kpad2 = pfn * rpp;
        if (MT * kpad2 > D3_AS || (kc >> 1) > (MT <= 2 ? 2 : 1) * D3_NT) continue;
        const int nslab = bo * nch * ks;
        if (nslab > resident - min_chain) continue;
        const double slab_bytes = (double)kc * lpr * 16.0;
        S1 t = {};
        if (!plan1(nslab, slab_bytes, t)) continue;
        const double t_slab = d3_stream_us(slab_bytes);
        const double t_z = t.t_chain + 2.2;
        const double est = (t_slab > t_z ? t_slab : t_z) + 0.8 + (ks > 1 ? 0.8 : 0.0) + (lpr < 16 ? (lpr < 8 ? 0.4 : 0.15) : 0.0);
        if (est < best) {
          best = est; found = true; s1 = t;
          p.lpr2_log2 = ilog2(lpr); p.nch2 = fd_make((uint32_t)nch); p.ks2 = ks; p.kc2 = kc; p.items2 = nslab; p.pfn = pfn; p.kpad2 = kpad2;
        }
      }
    }
    if (!found) return d2_bail(__LINE__);
  }
  p.bodiv = fd_make((uint32_t)bo);
  p.lpr1_log2 = ilog2(s1.lpr); p.nch1 = fd_make((uint32_t)s1.nch); p.bdiv = fd_make((uint32_t)b);
  p.ks1 = s1.ks; p.kc1 = s1.kc; p.nb1 = s1.nb; p.kpad1_log2 = ilog2(s1.kpad); p.items1 = s1.items; p.nchain = s1.nchain;
  if ((1 << p.kpad1_log2) != s1.kpad) return d2_bail(__LINE__);
  {
    int kld = 1;
    while (kld < p.kpad2) kld <<= 1;
    if (MT * kld > D3_AS) return d2_bail(__LINE__);
    p.kld2_log2 = ilog2(kld);
  }
  {
    // the speculative fetch of z pays when the chain is expected to deliver before the last eight loads of a slab land
    const double t_z = s1.t_chain + 2.2;
    const double slab_bytes = (double)p.kc2 * (1 << p.lpr2_log2) * 16.0;
    const double t_a = d3_stream_us(slab_bytes * (p.pfn > D3_PFB ? (double)(p.pfn - D3_PFB) / p.pfn : 0.0));
    p.zspec = (p.pfn > D3_PFB && t_z + 0.5 < t_a) ? 1 : 0;
  }

  const size_t ybytes = align_up((size_t)p.ks1 * b * M * R * 8, 256), zbytes = align_up((size_t)(p.zrep > 1 ? p.zrep : bo) * M * R * 8, 256);
  const size_t obytes = (size_t)(p.ks2 - 1) * bo * M * Q * 8;
  if (ybytes + zbytes + obytes > decode2_region_bytes()) return d2_bail(__LINE__);
  p.ypart = reinterpret_cast<unsigned long long*>(region);
  p.zt = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes);
  p.opart = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes + zbytes);
  p.epoch_word = epoch_word; p.arrive_word = arrive_word; p.err_word = err_word;
  const int grid = p.items2 + p.nchain;
  if (grid > resident) return d2_bail(__LINE__);
  static const int dbg = env_i("BLR_D2_DEBUG", 0);
  if (dbg) fprintf(stderr, "decode3: M=%d b=%d bo=%d P=%d R=%d Q=%d wb=%d | slabs %d (lpr %d, nch %u, ks %d, kc %d, pfn %d, zspec %d) chain %d (items %d, ks %d, kc %d, nb %d) mix %d\n",
                   M, b, bo, P, R, Q, WBITS, p.items2, 1 << p.lpr2_log2, p.nch2.d, p.ks2, p.kc2, p.pfn, p.zspec, p.nchain, p.items1, p.ks1, p.kc1, p.nb1, p.itemsM);
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3(grid), dim3(D3_NT), args, 0, st);
  if (e != hipSuccess) { set_error("decode3: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  if (p.ep) epilogue_taken();
  return BLR_OK;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace3(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace3), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

// BLAST at more than 16 rows, first half: Z = mix(S, x V) in one launch, with Y = x V never leaving the compute unit.
//
//   Z[i][m][r] = sum_j S(i, j, r) * Y_j[m][r],      Y_j = x_j V_j   (x_j: columns j P .. (j+1) P of x, V_j (P, R))
//
// The unfused path writes Y (b, M, R) to memory, reads it back in a mix kernel and writes Z: three passes over an
// intermediate that is larger than every operand.  Here a workgroup owns a tile of 32 rows x up to 128 ranks for ALL
// input blocks j and ALL output blocks i:
//   phase 1  each of the eight waves computes Y_j of the tile for two input blocks on the matrix cores.  V is row-major
//            (rank contiguous) and the matrix cores want eight consecutive k of one column per lane, so a lane loads its
//            16-byte piece of eight rows and product e takes element e of each (byte permutes; the column slots of
//            product e are the ranks 8 n + e).  Loads go straight to registers, two k-steps in flight.  The two Y_j of a
//            wave leave as (Y_2w, Y_2w+1) pairs of T, one dword per (m, r), into LDS.
//   phase 2  for one rank r the mix is a 16 x 16 matrix product over the input blocks, Z_r (i, m) = S_r (i, j) Y_r (j, m),
//            i.e. one matrix-core instruction per rank and 16 rows.  Its operands want four consecutive j per lane: Y
//            gives them as two of its pair dwords from LDS, S as eight contiguous bytes when it is stored (r, i, j) -
//            the layout of the bmm names; any other layout is transposed once per call into scratch by a small kernel.
//            A wave takes 16 ranks of the tile, keeps the products of eight ranks in registers and stores 16 bytes of
//            Z per (i, m).  Z leaves as T.
// What follows is an ordinary batched GEMM out_i = Z_i U_i.
#include <hip/hip_runtime.h>
#include <cmath>
#include "blr_common.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
constexpr int YM_NT = 512;
constexpr int YM_BM = 32;
constexpr uint32_t YM_OOB = 0x80000000u;
}  // namespace

#ifdef BLR_TRACE
__device__ unsigned long long g_trace6[1024 * 16];
#define TR6(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) g_trace6[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR6(i) do {} while (0)
#endif

struct YmixParams {
  const void* x; int64_t ldx; uint32_t x_bytes;
  const void* V; const void* S; void* Z;
  int M, b, P, R;
  int npc;                      // 16-byte rank pieces of a tile (1..16): the tile spans BR = 8 npc ranks
  int ksteps;                   // 32-row k-steps that cover P
  FastDiv nmt;                  // row tiles
  const void* St;               // S as (r, i, j), the input block contiguous
};

template <typename T> struct YmDot;
template <> struct YmDot<f16> {
  static __device__ __forceinline__ f32x4 mfma16(u32x2 a, u32x2 b, f32x4 c) {      // 16 x 16 x 16
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct YmDot<bf16> {
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ f32x4 mfma16(u32x2 a, u32x2 b, f32x4 c) {      // 16 x 16 x 16
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

template <typename T>
__device__ __forceinline__ uint32_t ym_pack(float lo, float hi) {
  typename TypeTraits<T>::vec4 v;      // (only two lanes used; a two-element vector of T has no common name here)
  v[0] = TypeTraits<T>::from_f32(lo); v[1] = TypeTraits<T>::from_f32(hi); v[2] = v[0]; v[3] = v[0];
  return __builtin_bit_cast(u32x2, v)[0];
}

template <typename T>
__global__ __launch_bounds__(YM_NT) void blast_ymix_kernel(YmixParams p) {
  extern __shared__ __attribute__((aligned(16))) uint32_t ym_lds[];
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
  const int b = p.b, P = p.P, R = p.R, M = p.M, BR = p.npc * 8, JP = b >> 1;
  // Y pairs (Y_2jp, Y_2jp+1) as [jp][m][r]: rows padded by 4 dwords and input-block planes by 16, so that the 16-byte
  // writes of phase 1 stay aligned and the reads of phase 2 (16 rows x 4 planes of one rank) spread over the banks
  const int RS = BR + 4, JS = YM_BM * RS + 16;
  uint32_t* y_s = ym_lds;
  // workgroups of one rank tile follow each other within an XCD: its slice of V stays in that L2 while the rows stream
  const uint32_t item = xcd_item(blockIdx.x, gridDim.x);
  const uint32_t rt = fd_div(item, p.nmt), mt = item - rt * p.nmt.d;
  const int m0 = (int)mt * YM_BM, r0 = (int)rt * BR;
  TR6(0);
  // the mix's S operands depend on nothing and are used after phase 1: asked for behind the first loads of phase 1 (the
  // memory pipeline takes an instruction every 16 cycles, and the products can only start on those first loads).  Lane (n, g)
  // of wave wv: S_r(i = n, j = 4 g .. 4 g + 3) for the wave's 16 ranks r0 + 16 wv ..; waves without ranks in the tile ask nothing
  const __amdgpu_buffer_rsrc_t sbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.St), 0, (uint32_t)((int64_t)b * b * R * 2), 0x00020000);
  const int rw = wv * 16;
  u32x2 sa[16];
  auto load_sa = [&]() {
    const bool a_ok = n < b && 4 * g < b;
    if (rw < BR) {
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int r = r0 + rw + q;
        const uint32_t off = (a_ok && rw + q < BR && r < R) ? (uint32_t)(((int64_t)r * b + n) * b + 4 * g) * 2u : YM_OOB;
        sa[q] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(sbuf, off, 0, 0));
      }
    }
  };

  // ---------------------------------------------- phase 1: Y pairs into LDS ----------------------------------------------
  // One pipeline over the k-steps of the wave's two input blocks (no drain between them): step q < KS belongs to block
  // 2 wv, step q >= KS to block 2 wv + 1; the accumulators of the first block are packed away at the boundary.
  if (wv < JP) {
    const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.x), 0, p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vbuf = wbuf(reinterpret_cast<const T*>(p.V) + (int64_t)(2 * wv) * P * R, (uint32_t)((int64_t)2 * P * R * 2));
    const bool live = n < p.npc && r0 + n * 8 < R;
    const int KS = p.ksteps;                                // 32-row steps per input block
    uint32_t h0[2][4][4];                                   // Y of the wave's first input block, packed two ranks to a dword
    f32x4 acc[2][8];
#pragma unroll
    for (int mg = 0; mg < 2; ++mg)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[mg][e] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 a0[2], a1[2], b0[8], b1[8];
    // step s of a block covers k = 32 s .. 32 s + 31; this lane holds k = 32 s + 8 g .. + 7 of row 16 mg + n (x) and of its
    // rank piece (V).  No branch around the loads (the compiler then waits for exactly the step it needs): what lies
    // outside - rows past M, k past P, lanes without a rank piece, steps past the second block - asks for an offset out
    // of bounds and reads zeros.
    auto load_ab = [&](u32x4 (&a)[2], u32x4 (&bb)[8], int q) {
      const int jj = q >= KS ? 1 : 0, sst = q - jj * KS;
      const int k = 32 * sst + 8 * g;
      const bool kin = k < P && q < 2 * KS;
#pragma unroll
      for (int mg = 0; mg < 2; ++mg) {
        const int m = m0 + 16 * mg + n;
        const uint32_t off = (m < M && kin) ? (uint32_t)((int64_t)m * p.ldx + (int64_t)(2 * wv + jj) * P + k) * 2u : YM_OOB;
        a[mg] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xbuf, off, 0, 0));
      }
      const uint32_t base = (live && kin) ? (uint32_t)((jj * P + k) * R + r0 + n * 8) * 2u : YM_OOB;
#pragma unroll
      for (int t = 0; t < 8; ++t) bb[t] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(vbuf, base + (uint32_t)(t * R) * 2u, 0, 0));
    };
    auto step = [&](const u32x4 (&a)[2], const u32x4 (&bb)[8]) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        u32x4 bv;
#pragma unroll
        for (int h = 0; h < 4; ++h) bv[h] = __builtin_amdgcn_perm(bb[2 * h + 1][e >> 1], bb[2 * h][e >> 1], sel);
#pragma unroll
        for (int mg = 0; mg < 2; ++mg) acc[mg][e] = YmDot<T>::mfma(a[mg], bv, acc[mg][e]);
      }
    };
    auto next_block = [&]() {                                // pack away the first block's Y, start the second from zero
#pragma unroll
      for (int mg = 0; mg < 2; ++mg)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int q = 0; q < 4; ++q) h0[mg][t][q] = ym_pack<T>(acc[mg][2 * q][t], acc[mg][2 * q + 1][t]);
#pragma unroll
      for (int mg = 0; mg < 2; ++mg)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[mg][e] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    load_ab(a0, b0, 0);
    load_sa();
    TR6(1);
    int q = 0;
    for (; q + 2 < 2 * KS; q += 2) {                         // two steps per trip (the two register sets take turns)
      if (q == KS) next_block();
      load_ab(a1, b1, q + 1);
      step(a0, b0);
      if (q + 1 == KS) next_block();
      load_ab(a0, b0, q + 2);
      step(a1, b1);
    }
    // the last trip on its own: nothing is left to ask for behind it (ten loads that would all be out of bounds still cost
    // their turns in the memory pipeline)
    if (q == KS) next_block();
    load_ab(a1, b1, q + 1);
    step(a0, b0);
    if (q + 1 == KS) next_block();
    step(a1, b1);
    TR6(2);
    // acc[mg][e][t] is Y of block 2 wv + 1 at [m0 + 16 mg + 4 g + t][r0 + 8 n + e]; h0 holds block 2 wv
    if (n < p.npc) {
#pragma unroll
      for (int mg = 0; mg < 2; ++mg)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          uint32_t pr[8];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t h1 = ym_pack<T>(acc[mg][2 * q][t], acc[mg][2 * q + 1][t]);
            pr[2 * q] = __builtin_amdgcn_perm(h1, h0[mg][t][q], 0x05040100u);          // rank 8 n + 2 q:     (Y_2w, Y_2w+1)
            pr[2 * q + 1] = __builtin_amdgcn_perm(h1, h0[mg][t][q], 0x07060302u);      // rank 8 n + 2 q + 1
          }
          uint32_t* dst = &y_s[wv * JS + (16 * mg + 4 * g + t) * RS + n * 8];
          *reinterpret_cast<u32x4*>(dst) = u32x4{pr[0], pr[1], pr[2], pr[3]};
          *reinterpret_cast<u32x4*>(dst + 4) = u32x4{pr[4], pr[5], pr[6], pr[7]};
        }
    }
  } else {
    load_sa();
  }
  TR6(3);
  __syncthreads();
  TR6(4);

  // ---------------------------------------------- phase 2: the mix ----------------------------------------------------------
  // lane (n, g): operand A = S_r(i = n, j = 4 g .. 4 g + 3), operand B = Y_r(j = 4 g .. 4 g + 3, m = 16 mg + n); the
  // product's lane holds Z_r(i = 4 g + t, m = 16 mg + n), t = 0..3
  if (rw < BR) {
    const bool b_ok = 2 * g < JP;
#pragma unroll
    for (int mg = 0; mg < 2; ++mg) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {                          // eight ranks at a time
        if (rw + 8 * h < BR) {
          f32x4 d[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int rr = rw + 8 * h + q;
            u32x2 yb = {0u, 0u};
            if (b_ok) {
              const uint32_t* src = &y_s[(2 * g) * JS + (16 * mg + n) * RS + rr];
              yb[0] = src[0]; yb[1] = src[JS];
            }
            d[q] = YmDot<T>::mfma16(sa[8 * h + q], yb, f32x4{0.f, 0.f, 0.f, 0.f});
          }
          const int m = m0 + 16 * mg + n, r = r0 + rw + 8 * h;
          if (m < M && r < R) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int i = 4 * g + t;
              if (i < b) {
                u32x4 o;
#pragma unroll
                for (int q = 0; q < 4; ++q) o[q] = ym_pack<T>(d[2 * q][t], d[2 * q + 1][t]);
                *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.Z) + ((int64_t)i * M + m) * R + r) = o;
              }
            }
          }
        }
      }
    }
  }
  TR6(14);
}

// S(i, j, r) with any strides -> St[(r b + i) b + j]: one thread per (i, r), neighbouring threads on neighbouring ranks.
template <typename T>
__global__ __launch_bounds__(256) void ym_s_transpose_kernel(const T* __restrict__ S, T* __restrict__ St, int b, int R,
                                                              int64_t s_si, int64_t s_sj, int64_t s_sr) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= b * R) return;
  const int r = idx % R, i = idx / R;
  for (int j = 0; j < b; ++j) St[((int64_t)r * b + i) * b + j] = S[(int64_t)i * s_si + (int64_t)j * s_sj + (int64_t)r * s_sr];
}

// Z (b, M, R) of dtype = mix(S, x V).  scratch: room for S transposed to (r, i, j) (b b R elements), used unless S already
// has that layout.  Returns BLR_OK, a negative blr_status, or 1 when the shape is not for this kernel (b not a multiple of
// 4 or above 16, rank or block width not a multiple of 8, unaligned operands, fp32, scratch too small).
int blast_ymix_launch(const void* x, int64_t ldx, const void* V, const void* S, void* Z, int M, int in_f, int b, int R,
                      int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                      hipStream_t st) {
  if (dtype != BLR_F16 && dtype != BLR_BF16) return 1;
  if (b < 4 || b > 16 || (b & 3) || in_f % b) return 1;
  const int P = in_f / b;
  if (P % 8 || R % 8 || ldx % 8 || !aligned(x, 16) || !aligned(V, 16) || !aligned(Z, 16)) return 1;
  const int64_t x_elems = (int64_t)(M - 1) * ldx + in_f;
  if (x_elems * 2 >= (int64_t)YM_OOB || (int64_t)P * R * 2 >= (int64_t)YM_OOB || (int64_t)b * b * R * 2 >= (int64_t)YM_OOB) return 1;
  YmixParams p = {};
  p.x = x; p.ldx = ldx; p.x_bytes = (uint32_t)(x_elems * 2); p.V = V; p.S = S; p.Z = Z;
  p.M = M; p.b = b; p.P = P; p.R = R;
  // Rank pieces per tile.  One workgroup per compute unit at a time; a workgroup takes about 10 + 0.85 npc us at 72-column input
  // blocks, i.e. 12 + npc units, and a last round that is not full costs about half of what it leaves empty.  Measured at 4096
  // rows, r = 576: 15 pieces = 640 workgroups (2.5 rounds) 68 us, 12 = 768 (3 rounds) 60 us, 9 = 1024 (4 rounds) 72 us; r = 288:
  // 12 pieces = 384 (1.5 rounds) 34.8 us, 9 = 512 (2 rounds) 36.2 us.
  const int pieces = R / 8;
  const int cus = device_cus() > 0 ? device_cus() : 256;
  static const int e_npc = env_i("BLR_YM_NPC", 0);
  int best_npc = 16; double best_cost = -1.0;
  for (int npc = 16; npc >= 4; --npc) {
    const double x = (double)(cdiv(pieces, npc) * cdiv(M, YM_BM)) / cus;
    const double cost = 0.5 * (std::ceil(x) + x) * (12 + npc);
    if (best_cost < 0 || cost < best_cost - 1e-9) { best_cost = cost; best_npc = npc; }
  }
  p.npc = e_npc > 0 && e_npc <= 16 ? e_npc : best_npc;
  const int nrt = (int)cdiv(pieces, p.npc), nmt = (int)cdiv(M, YM_BM);
  if ((int64_t)nrt * nmt >= 65536 || nmt >= 65536) return 1;
  p.nmt = fd_make((uint32_t)nmt);
  p.ksteps = (int)cdiv(P, 32);
  if (s_layout == BLR_S_RIJ && aligned(S, 8)) {
    p.St = S;
  } else {
    if (!scratch || scratch_bytes < (size_t)b * b * R * 2 || !aligned(scratch, 8)) return 1;
    const unsigned tg = (unsigned)cdiv((int64_t)b * R, 256);
    if (dtype == BLR_F16) hipLaunchKernelGGL(ym_s_transpose_kernel<f16>, dim3(tg), dim3(256), 0, st, (const f16*)S, (f16*)scratch, b, R, s_si, s_sj, s_sr);
    else hipLaunchKernelGGL(ym_s_transpose_kernel<bf16>, dim3(tg), dim3(256), 0, st, (const bf16*)S, (bf16*)scratch, b, R, s_si, s_sj, s_sr);
    BLR_CHECK_LAUNCH("ym_s_transpose");
    p.St = scratch;
  }
  const int BR = p.npc * 8;
  const size_t lds = (size_t)(b / 2) * (YM_BM * (BR + 4) + 16) * 4;
  void* fn = dtype == BLR_F16 ? (void*)blast_ymix_kernel<f16> : (void*)blast_ymix_kernel<bf16>;
  static bool attr_set[2] = {false, false};
  if (!attr_set[dtype == BLR_F16 ? 0 : 1]) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) { set_error("blast_ymix: cannot raise the LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    attr_set[dtype == BLR_F16 ? 0 : 1] = true;
  }
  const dim3 grid((unsigned)(nrt * nmt)), block(YM_NT);
  if (dtype == BLR_F16) hipLaunchKernelGGL(blast_ymix_kernel<f16>, grid, block, lds, st, p);
  else hipLaunchKernelGGL(blast_ymix_kernel<bf16>, grid, block, lds, st, p);
  BLR_CHECK_LAUNCH("blast_ymix");
  return BLR_OK;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace6(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace6), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

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
#include <type_traits>
#include "blr_common.h"
#include "blr_decode_dev.h"
#include "blr_ring_dev.h"

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

template <typename T, bool STAGE>
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
  // A lane's 16 bytes of Z belong to a row (i, m) of their own: stored from here, an instruction touches 64 cache lines and
  // holds the memory pipeline eight times as long as one that writes whole rows (5.3 of a workgroup's 15 us were these
  // stores).  STAGE: the 16 rows of a product group go through LDS behind Y ([i][m][rank], 16 lanes per row) and leave as
  // runs of BR ranks; without (the tile's Y leaves no room for that) the lanes store their pieces themselves.
  const bool b_ok = 2 * g < JP;
  const int ZRS = BR / 2 + 4;                                // dwords per staged row
  uint32_t* const z_st = ym_lds + JP * JS;
#pragma unroll
  for (int mg = 0; mg < 2; ++mg) {
    if (STAGE && mg == 1) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // the first group's rows have been read
    if (rw < BR) {
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
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int i = 4 * g + t;
            u32x4 o;
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = ym_pack<T>(d[2 * q][t], d[2 * q + 1][t]);
            if (STAGE) {
              if (i < b) *reinterpret_cast<u32x4*>(&z_st[(i * 16 + n) * ZRS + (rw + 8 * h) / 2]) = o;
            } else if (m < M && r < R && i < b) {
              *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.Z) + ((int64_t)i * M + m) * R + r) = o;
            }
          }
        }
      }
    }
    if (STAGE) {
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      const int pc = tid & 15, r = r0 + pc * 8;
      if (pc < p.npc && r < R) {                           // 32 rows per pass: output blocks 2 it, 2 it + 1
        const int rr = tid >> 4, m = m0 + 16 * mg + (rr & 15);
        u32x4 v[8];
#pragma unroll
        for (int it = 0; it < 8; ++it)
          if (2 * it < b) v[it] = *reinterpret_cast<const u32x4*>(&z_st[(rr + 32 * it) * ZRS + pc * 4]);
        if (m < M) {
#pragma unroll
          for (int it = 0; it < 8; ++it)
            if (2 * it + (rr >> 4) < b) *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.Z) + ((int64_t)(2 * it + (rr >> 4)) * M + m) * R + r) = v[it];
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
  int best_npc = 16; double best_cost = -1.0;
  for (int npc = 16; npc >= 4; --npc) {
    const double x = (double)(cdiv(pieces, npc) * cdiv(M, YM_BM)) / cus;
    const double cost = 0.5 * (std::ceil(x) + x) * (12 + npc);
    if (best_cost < 0 || cost < best_cost - 1e-9) { best_cost = cost; best_npc = npc; }
  }
  p.npc = best_npc;
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
  const size_t lds_y = (size_t)(b / 2) * (YM_BM * (BR + 4) + 16) * 4;
  const size_t lds_z = (size_t)b * 16 * (BR / 2 + 4) * 4;                 // the rows of one product group on their way out
  const bool stage = lds_y + lds_z <= 160 * 1024;
  const size_t lds = lds_y + (stage ? lds_z : 0);
  const int fi = (dtype == BLR_F16 ? 0 : 2) + (stage ? 1 : 0);
  void* const fns[4] = {(void*)blast_ymix_kernel<f16, false>, (void*)blast_ymix_kernel<f16, true>,
                        (void*)blast_ymix_kernel<bf16, false>, (void*)blast_ymix_kernel<bf16, true>};
  static bool attr_set[4] = {false, false, false, false};
  if (!attr_set[fi]) {
    hipError_t e = hipFuncSetAttribute(fns[fi], hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) { set_error("blast_ymix: cannot raise the LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    attr_set[fi] = true;
  }
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fns[fi], dim3((unsigned)(nrt * nmt)), dim3(YM_NT), args, lds, st);
  if (e != hipSuccess) { set_error("blast_ymix: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}


// ---- the same first half for wide input blocks: x V as one GEMM over all of x's columns, Y held in registers -------------------
//
// blast_ymix_kernel reads V once per 32 rows, straight into registers; from about 128 columns per input block on that costs more
// than the round trip of Y through memory that it saves.  Here a workgroup of four waves (one per SIMD, so a lane may hold some
// 250 registers) owns 64 rows x 64 ranks for all 16 input blocks.  x is (M, 16 P) and V (16 P, R), both contiguous over the
// blocks, so Y_0 .. Y_15 of the tile are one GEMM with a reduction over all 16 P columns whose accumulator is packed away and
// cleared every P columns: stages of 64 k of both operands go global -> LDS directly (whole 128-byte lines; the stage layouts
// and fragment reads of gemm_ring64_kernel), YW_NST stages deep, one barrier per stage; a wave's 32 x 32 block of Y_j leaves the
// accumulator as 8 dwords (two ranks each), 128 dwords for the sixteen blocks.  When the reduction is done the ring is no longer
// needed: Y goes to LDS as dwords (Y_2jp, Y_2jp+1) [jp][row][rank ^ f(row, jp)], and the mix runs as in blast_ymix_kernel (one
// 16 x 16 x 16 matrix instruction per rank and 16 rows), its rows of Z staged through LDS and stored as whole 128-byte lines.
namespace {
constexpr int YW_NT = 256, YW_NST = 8, YW_STG = 8192;      // threads; ring depth; bytes of a stage of one operand (64 x 64 elements)
constexpr size_t YW_LDS = 160 * 1024;                      // ring: 2 x 8 x 8 KiB + the tile's slice of S 32 KiB; afterwards Y 128 KiB + staged rows of Z 32 KiB
}

struct YmixwParams {
  const void* x; int64_t ldx;
  const void* V; const void* St; void* Z;
  int M, R, KT;                 // KT: stages of 64 k per input block (P / 64)
  FastDiv nrt;                  // rank tiles
  int s_stage;                  // 0: St is S as (r, i, j), read straight into the mix's operands; 1: S has the rank contiguous
  int64_t s_si, s_sj;           //    (strides of i and j in elements): the tile's slice goes through LDS
};

template <typename T>
__global__ __launch_bounds__(YW_NT, 1) void blast_ymixw_kernel(YmixwParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char yw_lds[];
  constexpr int NWV = 4, NST = YW_NST, BRING = NST * YW_STG, LT = 4, RB = 128;
  using V8 = typename TypeTraits<T>::vec8;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int M = p.M, R = p.R;
  // a run of items per XCD, rank tiles fastest: the workgroups of an XCD at any time share two tiles of rows of x in its L2
  const uint32_t item = xcd_item(blockIdx.x, gridDim.x);
  const uint32_t mt = fd_div(item, p.nrt), rt = item - mt * p.nrt.d;
  const int m0 = (int)mt * 64, r0 = (int)rt * 64;
  TR6(0);
  const int n = lane & 15, g = lane >> 4, rw = wave * 16;
  // ---------------------------------------------- phase 1: Y of the tile, in registers --------------------------------------
  // stage s covers columns 64 s .. 64 s + 63 of x and rows 64 s .. of V (all blocks).  K-contiguous stage (x): a load takes eight
  // 16-byte chunks of each of 8 rows, lane (r8, s8) chunk s8 ^ r8; (k, n) stage (V): a load takes 8 rows of 64 ranks, chunk c of
  // row k stored at c ^ ((k & 3) << 1).
  const int r8 = lane >> 3, s8 = lane & 7, c8 = s8 ^ r8;
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    a_off[i] = (uint32_t)(min(m0 + (i * NWV + wave) * 8 + r8, M - 1) * p.ldx * 2 + c8 * 16);
    const int krow = (i * NWV + wave) * 8 + r8;
    b_off[i] = (uint32_t)((krow * R + r0 + (s8 ^ ((krow & 3) << 1)) * 8) * 2);
  }
  const uint32_t lds0 = ring_lds_addr(yw_lds + wave * 1024);
  const char* Ab = reinterpret_cast<const char*>(p.x);
  const char* Bb = reinterpret_cast<const char*>(p.V);
  auto issue = [&](int s, int slot) {
    const char* ap = Ab + (int64_t)s * 128;
    const char* bp = Bb + (int64_t)s * 64 * R * 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) ring_load_lds(ap, a_off[i], lds0 + slot * YW_STG + i * (NWV * 1024));
#pragma unroll
    for (int i = 0; i < 2; ++i) ring_load_lds(bp, b_off[i], lds0 + BRING + slot * YW_STG + i * (NWV * 1024));
  };
  const int half = lane >> 5;
  const int rl = wm * 32 + (lane & 31);
  const uint32_t rowA = (uint32_t)(((rl >> 3) << 10) + ((rl & 7) << 7));
  uint32_t xo[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) xo[q] = (uint32_t)(((2 * q + half) ^ (lane & 7)) << 4);
  const int i16 = lane & 15;
  const int chunk0 = wn * 4 + (g & 1) * 2 + ((i16 & 3) >> 1);
  const uint32_t rowB = (uint32_t)(((g >> 1) * 8 + (i16 >> 2)) * RB + (i16 & 1) * 8 + ((chunk0 ^ ((i16 >> 2) << 1)) << 4));

  // Stage t lives in slot t % NST; NST - 1 stages are in flight.  A stage takes about 620 cycles here whatever the order of the
  // loop: the same with every workgroup of the launch on one and the same tile (all loads L2 hits), with a ring of ten stages,
  // with two accumulators taking the sub-steps in turn and with the fragments of stage s + 1 read under the products of stage s
  // (the blocks of Y pinned to accumulation registers to make room) - in-kernel cycle counts then show 29 % of a wave's loop in
  // the issue of its four loads: the compute unit's sixteen load instructions and 48 KiB of LDS traffic per stage are what a
  // 64 x 64 tile costs, and the tile cannot grow because Y of sixteen blocks has to stay in registers.  (Asking for every line a
  // first time twenty stages early, by a 4-byte load per line into a dump area, made it slower: 18.5 -> 28.9 us per tile at
  // P = 256, R = 512 - an instruction that touches 32 lines costs the address path as much as four that fetch them.)
  const int s_total = 16 * p.KT;
#pragma unroll
  for (int s = 0; s < NST - 1; ++s) issue(min(s, s_total - 1), s);
  TR6(1);
  // S with the rank contiguous ((j, i, r) or (i, j, r)): the 256 rows (j, i) x 64 ranks of this tile go to LDS behind the ring,
  // where nothing else lives until the mix stages its rows of Z - by then the operands are in registers
  T* const s_t = reinterpret_cast<T*>(yw_lds + 2 * YW_NST * YW_STG);
  if (p.s_stage) {
    const T* Sg = reinterpret_cast<const T*>(p.St);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = it * YW_NT + tid, ji = idx >> 3, c = (idx & 7) * 8;
      *reinterpret_cast<V8*>(&s_t[ji * 64 + c]) = *reinterpret_cast<const V8*>(&Sg[(int64_t)(ji & 15) * p.s_si + (int64_t)(ji >> 4) * p.s_sj + r0 + c]);
    }
  }

  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
  uint32_t yreg[16][8];
  int s = 0, slot = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    for (int kt = 0; kt < p.KT; ++kt, ++s) {
      __builtin_amdgcn_s_waitcnt(ring_vmcnt((NST - 2) * LT));   // this wave's part of stage s has landed
      __builtin_amdgcn_s_barrier();                             // everybody's has, and nobody reads stage s - 1 any more
      issue(min(s + NST - 1, s_total - 1), slot == 0 ? NST - 1 : slot - 1);   // (past the end: the last stage again, never read)
      const unsigned char* sta = yw_lds + slot * YW_STG;
      const unsigned char* stb = yw_lds + BRING + slot * YW_STG;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const V8 af = *reinterpret_cast<const V8*>(sta + rowA + xo[q]);
        union { V8 v; s16x4 h[2]; } w;
        w.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(stb + rowB + (q * 16) * RB));
        w.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(stb + rowB + (q * 16 + 4) * RB));
        acc = TypeTraits<T>::mfma32(w.v, af, acc);             // (ranks as rows: the product comes out transposed)
      }
      slot = slot + 1 == NST ? 0 : slot + 1;
    }
    // acc[4 q + e] is Y_j at row wm 32 + (lane & 31), rank wn 32 + 8 q + 4 half + e
#pragma unroll
    for (int d = 0; d < 8; ++d) yreg[j][d] = ym_pack<T>(acc[2 * d], acc[2 * d + 1]);
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
  }
  TR6(2);
  __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));                    // the repeats of the last stage have landed too: the ring is free
  __builtin_amdgcn_s_barrier();
  // the mix's S operands, asked for now (the loop had no registers to spare) and used after Y has gone to LDS.  Lane (n, g) of
  // wave w: S_r(i = n, j = 4 g .. 4 g + 3), r = r0 + 16 w ..
  u32x2 sa[16];
  if (p.s_stage) {                                              // (the barrier above is behind every wave's stores of the slice)
    const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s_t);
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      uint32_t v[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) v[jj] = s16[((4 * g + jj) * 16 + n) * 64 + rw + q];
      sa[q] = u32x2{v[0] | (v[1] << 16), v[2] | (v[3] << 16)};
    }
  } else {
    const __amdgpu_buffer_rsrc_t sbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.St), 0, (uint32_t)((int64_t)256 * R * 2), 0x00020000);
#pragma unroll
    for (int q = 0; q < 16; ++q)
      sa[q] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(sbuf, (uint32_t)(((r0 + rw + q) * 16 + n) * 16 + 4 * g) * 2u, 0, 0));
  }

  // Y -> LDS: dword (Y_2jp, Y_2jp+1) of (row m, rank r) at [jp][m][r ^ ((m & 15) + 16 (jp >> 1))] - the 64 lanes of a mix read
  // (16 rows x 4 pairs of planes, one rank) then hit 64 different banks.  Dword d of a block holds ranks ra, ra + 1 (ra even):
  // neighbours in LDS, in the order the row's parity gives.
  uint32_t* const y_s = reinterpret_cast<uint32_t*>(yw_lds);
  {
    const int m = wm * 32 + (lane & 31);
#pragma unroll
    for (int jp = 0; jp < 8; ++jp)
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        const uint32_t h0 = yreg[2 * jp][d], h1 = yreg[2 * jp + 1][d];
        const uint32_t da = __builtin_amdgcn_perm(h1, h0, 0x05040100u), db = __builtin_amdgcn_perm(h1, h0, 0x07060302u);
        const int ra = wn * 32 + 8 * (d >> 1) + 4 * half + 2 * (d & 1);
        const int col = (ra ^ ((m & 15) + 16 * (jp >> 1))) & ~1;
        *reinterpret_cast<u32x2*>(&y_s[jp * 4096 + m * 64 + col]) = (m & 1) ? u32x2{db, da} : u32x2{da, db};
        if (d == 7) __builtin_amdgcn_sched_barrier(0);          // (one pair of blocks at a time: nothing to gain from more in flight)
      }
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  TR6(3); TR6(4);

  // ---------------------------------------------- phase 2: the mix --------------------------------------------------------
  // lane (n, g): operand A = S_r(i = n, j = 4 g .. 4 g + 3), operand B = Y_r(j = 4 g .. 4 g + 3, m = 16 mg + n); the product's lane
  // holds Z_r(i = 4 g + t, m = 16 mg + n).  The 256 rows (i, m) of a group of 16 rows of the tile go through LDS (128 bytes each,
  // 16-byte slots XOR-ed with the row's low bits) and leave as whole lines.
  uint32_t* const z_st = y_s + 8 * 4096;
#pragma unroll 1
  for (int mg = 0; mg < 4; ++mg) {
    if (mg) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // the previous group's rows have been read
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 d[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int rr = rw + 8 * h + q;
        const uint32_t* src = &y_s[(2 * g) * 4096 + (16 * mg + n) * 64 + (rr ^ (n + 16 * g))];
        const u32x2 yb = {src[0], src[4096]};
        d[q] = YmDot<T>::mfma16(sa[8 * h + q], yb, f32x4{0.f, 0.f, 0.f, 0.f});
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        u32x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = ym_pack<T>(d[2 * q][t], d[2 * q + 1][t]);
        const int row = (4 * g + t) * 16 + n;
        *reinterpret_cast<u32x4*>(&z_st[row * 32 + (((wave * 2 + h) ^ (row & 7)) << 2)]) = o;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    {
      const int pc = tid & 7, rr = tid >> 3;               // 16-byte piece of a row; rows rr, rr + 32, ...
      u32x4 v[8];
#pragma unroll
      for (int it = 0; it < 8; ++it) v[it] = *reinterpret_cast<const u32x4*>(&z_st[(rr + 32 * it) * 32 + ((pc ^ (rr & 7)) << 2)]);
      const int m = m0 + 16 * mg + (rr & 15);
      if (m < M) {
#pragma unroll
        for (int it = 0; it < 8; ++it)
          *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.Z) + ((int64_t)(2 * it + (rr >> 4)) * M + m) * R + r0 + pc * 8) = v[it];
      }
    }
  }
  TR6(14);
}

// Z (16, M, R) of dtype = mix(S, x V) for 16 input blocks of a multiple of 64 columns and a rank that is a multiple of 64.
// scratch: room for S transposed to (r, i, j), used unless S already has that layout.  Returns BLR_OK, a negative blr_status, or
// 1 when the shape is not for this kernel.
int blast_ymixw_launch(const void* x, int64_t ldx, const void* V, const void* S, void* Z, int M, int in_f, int b, int R,
                       int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                       hipStream_t st) {
  if (dtype != BLR_F16 && dtype != BLR_BF16) return 1;
  if (b != 16 || in_f % 16) return 1;
  const int P = in_f / 16;
  if (P % 64 || R % 64 || ldx % 8 || !aligned(x, 16) || !aligned(V, 16) || !aligned(Z, 16)) return 1;
  if (((int64_t)(M - 1) * ldx + in_f) * 2 >= ((int64_t)1 << 31) || (int64_t)64 * R * 2 >= ((int64_t)1 << 31) || (int64_t)256 * R * 2 >= ((int64_t)1 << 31)) return 1;
  // (A variant with 64 rows x 128 ranks on eight waves - two per SIMD, three quarters of the operand bytes per product, the tile's
  // two halves of 64 ranks mixed one after the other - passed the same tests and measured slower: a stage of its loop took 575 ns
  // against 270 ns, 4096 -> 22016 at 2048 rows 177 against 173 us for the call.  The same tile on four waves - a wave holding 32 rows
  // x 64 ranks, its 256 dwords of Y spilling over into the accumulation registers, a ring of four stages of 24 KiB, the mix a quarter
  // of the tile at a time - was no better: 39.2 us in the loop for twice the products of the 17.3 us here, 30 us in the mix against
  // 2 x 6.8, the call 177.5 against 171.7 us.  Fewer load instructions per product do not speed this loop up.)
  const int nmt = (int)cdiv(M, 64), nrt = R / 64;
  if ((int64_t)nmt * nrt >= 65536) return 1;
  YmixwParams p = {};
  p.x = x; p.ldx = ldx; p.V = V; p.Z = Z; p.M = M; p.R = R; p.KT = P / 64;
  p.nrt = fd_make((uint32_t)nrt);
  if (s_layout == BLR_S_RIJ && aligned(S, 8)) {
    p.St = S;
  } else if (s_sr == 1 && s_si % 8 == 0 && s_sj % 8 == 0 && aligned(S, 16)) {
    p.St = S; p.s_stage = 1; p.s_si = s_si; p.s_sj = s_sj;
  } else {
    if (!scratch || scratch_bytes < (size_t)256 * R * 2 || !aligned(scratch, 8)) return 1;
    const unsigned tg = (unsigned)cdiv((int64_t)16 * R, 256);
    if (dtype == BLR_F16) hipLaunchKernelGGL(ym_s_transpose_kernel<f16>, dim3(tg), dim3(256), 0, st, (const f16*)S, (f16*)scratch, 16, R, s_si, s_sj, s_sr);
    else hipLaunchKernelGGL(ym_s_transpose_kernel<bf16>, dim3(tg), dim3(256), 0, st, (const bf16*)S, (bf16*)scratch, 16, R, s_si, s_sj, s_sr);
    BLR_CHECK_LAUNCH("ym_s_transpose");
    p.St = scratch;
  }
  void* const fn = dtype == BLR_F16 ? (void*)blast_ymixw_kernel<f16> : (void*)blast_ymixw_kernel<bf16>;
  static bool attr_set[2] = {false, false};
  if (!attr_set[dtype == BLR_F16 ? 0 : 1]) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)YW_LDS);
    if (e != hipSuccess) { set_error("blast_ymixw: cannot raise the LDS limit: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    attr_set[dtype == BLR_F16 ? 0 : 1] = true;
  }
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3((unsigned)(nmt * nrt)), dim3(YW_NT), args, YW_LDS, st);
  if (e != hipSuccess) { set_error("blast_ymixw: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}


// ---- second half for narrow output blocks: out_i = mix(S, Y)_i U_i in one launch, Z never written -------------------------
//
// When an output block is at most 80 columns wide, the results of ALL output blocks for a tile of 16 rows fit the registers of one
// workgroup (16 blocks x 16 rows x 80 columns of fp32 = 80 KB).  The workgroup then walks the rank in blocks of 64: it reads the
// block of Y for all input blocks once (the only pass over the intermediate), forms the block of every Z_i on the matrix cores
// (one 16 x 16 x 16 product per rank, as in the kernel above), hands it through LDS as T and multiplies it with the block of U_i.
// U (b, Q, R) has the rank contiguous, so 16 bytes of it are an operand as they stand - but the lanes of a matrix-core operand
// are its rows, and a load whose neighbouring lanes read different rows of U occupies the compute unit's memory pipeline for 64
// cycles instead of 16 (measured: 3 us per step with such loads, 0.5 us without any).  A small kernel therefore first re-lays U
// (1.3 MB at 4608 -> 1152, rank 576) and S in the order the lanes read them: U as (i, rank / 8, q, 8) - neighbouring lanes, i.e.
// neighbouring columns q, then read neighbouring 16-byte pieces - and S as (r / 2, j / 4, i, r % 2, 4), 16 bytes per lane and pair of ranks.
// A block of 64 ranks is two matrix-core steps of 32; step s takes the ranks 16 g + 8 s + e (g = 0..3 the lane group, e = 0..7 the
// element of the lane's 16 bytes).
//   wave w: four of the 32 load instructions that bring a block of Y (8 rows of 128 bytes each) into LDS; the mix of slots
//   4 w .. 4 w + 3 of a step (ranks 16 (w / 2) + 8 s + 4 (w % 2) + 0..3 of the block); output blocks 2 w, 2 w + 1.
// S and U of step c + 2 are asked for right after step c has used its registers, Y of the next block at the start of a block.
namespace {
constexpr int MU_NT = 512;
constexpr int MU_BM = 16;
constexpr int MU_RB = 64;       // ranks per block
constexpr int MU_LDY = 72;      // two-byte elements per LDS row of Y (64 ranks): 144 bytes keep 16-byte accesses aligned and rows apart
constexpr int MU_LDZ = 40;      // per LDS row of Z (the 32 slots of a step)
__device__ __forceinline__ void mu_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
}  // namespace

struct MixuParams {
  const void* Y; const void* Sp; const void* Ut; void* out; int64_t ldo;     // Sp (r / 2, j / 4, i, r % 2, 4), Ut (i, rank / 8, q, 8)
  int M, R, Q;
  uint32_t y_bytes;
  int rotate;
  const void* bias; int act;
  const void* gate; int gate_rows; int64_t ld_gate;
  const void* resid; int64_t ld_resid;
};

template <typename T, int NTQ>
__global__ __launch_bounds__(MU_NT) void blast_mixu_kernel(MixuParams p) {
  __shared__ __attribute__((aligned(16))) uint16_t mu_lds[256 * MU_LDY + 2 * 256 * MU_LDZ];
  uint16_t* const y_s = mu_lds;                              // [input block j][row m][rank of the block]
  uint16_t (*const z_s)[256 * MU_LDZ] = reinterpret_cast<uint16_t (*)[256 * MU_LDZ]>(mu_lds + 256 * MU_LDY);   // per step: [output block i][row m][slot]
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
  const int M = p.M, R = p.R, Q = p.Q;
  const int m0 = (int)blockIdx.x * MU_BM;
  const int NB = (R + MU_RB - 1) / MU_RB;             // the last block may hold 32 ranks: what lies past them is not asked for
  const bool half_u = (R % MU_RB) != 0 && g >= 2, half_y = (R % MU_RB) != 0 && (l & 7) >= 4;
  // Workgroups walk the blocks of ranks in turn from different starting points: all of them read the same ranks of U and S
  // otherwise, at the same moment, from the same lines of the eight L2s.  (The sum over the blocks is in fp32 and its order is
  // fixed per row tile.)
  const int rot = p.rotate ? (int)(blockIdx.x % (unsigned)NB) : 0;
  auto blk = [&](int k) { const int kk = k + rot; return kk >= NB ? kk - NB : kk; };
  TR6(0);
  const __amdgpu_buffer_rsrc_t ybuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Y), 0, p.y_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t sbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Sp), 0, (uint32_t)(256 * R * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t ubuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Ut), 0, (uint32_t)((int64_t)16 * Q * R * 2), 0x00020000);
  // Y: eight lanes fetch the 128 bytes of one (j, m); a load instruction covers eight rows m of one input block; the wave's four
  // loads are rows 0..7 and 8..15 of the input blocks 2 wv and 2 wv + 1.  Per-lane offsets are few (registers are short):
  // whatever is the same for all lanes goes into the scalar offset of the load.
  const int piece = l & 7, yrow = l >> 3;
  uint32_t yoff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    yoff[h] = m0 + 8 * h + yrow < M ? (uint32_t)(((int64_t)(2 * wv) * M + m0 + 8 * h + yrow) * R + piece * 8) * 2u : YM_OOB;
  const uint32_t yjs = (uint32_t)((int64_t)M * R * 2);           // from one input block to the next
  const int ypos = ((2 * wv) * 16 + yrow) * MU_LDY + piece * 8;
  // S_r(i = n, j = 4 g .. 4 g + 3) of the wave's four ranks of a step
  const int rk = 16 * (wv >> 1) + 4 * (wv & 1);                  // + 8 s + 64 k
  const uint32_t soff = (uint32_t)((rk >> 1) * 64 + l) * 16u;      // Sp: 16 bytes per lane and pair of ranks
  // U_i(q = 16 nt + n, ranks 16 g + 8 s .. + 7 of the block), i = 2 wv + ii: piece (i, 8 k + 2 g + s, q) of Ut
  const uint32_t uoff = (uint32_t)(((int64_t)(2 * wv) * (R / 8) + 2 * g) * Q + n) * 16u;
  const uint32_t uoff_last = 16 * (NTQ - 1) + n < Q ? uoff : YM_OOB;      // the last column tile of a block may be partly empty
  const uint32_t uis = (uint32_t)((R / 8) * Q) * 16u;            // from one output block to the next
  struct Regs { u32x4 s[2]; u32x4 u[2][NTQ]; };
  auto load_y = [&](u32x4 (&yr)[4], int k) {
    const bool cut = half_y && k == NB - 1;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      yr[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ybuf, cut ? YM_OOB : yoff[u & 1], (uint32_t)k * (MU_RB * 2u) + (uint32_t)(u >> 1) * yjs, 0));
  };
  auto store_y = [&](const u32x4 (&yr)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) *reinterpret_cast<u32x4*>(&y_s[ypos + ((u >> 1) * 16 + (u & 1) * 8) * MU_LDY]) = yr[u];
  };
  auto load_s = [&](Regs& r, int k, int s) {                 // rank 64 k + 8 s + rk + q
#pragma unroll
    for (int q = 0; q < 2; ++q) r.s[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, soff + (uint32_t)q * 1024u, (uint32_t)(k * MU_RB + 8 * s) * 512u, 0));
  };
  auto load_u = [&](Regs& r, int k, int s) {
    const bool cut = half_u && k == NB - 1;
    const uint32_t v0 = cut ? YM_OOB : uoff, vl = cut ? YM_OOB : uoff_last;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
      for (int nt = 0; nt < NTQ; ++nt)
        r.u[ii][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ubuf, (nt == NTQ - 1 ? vl : v0) + (uint32_t)nt * 256u,
                                                                                        (uint32_t)((8 * k + s) * Q) * 16u + (uint32_t)ii * uis, 0));
  };
  f32x4 acc[2][NTQ];
#pragma unroll
  for (int ii = 0; ii < 2; ++ii)
#pragma unroll
    for (int nt = 0; nt < NTQ; ++nt) acc[ii][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // step s of block k on the register set `cur`.  No load sits under a condition (the compiler would then wait for everything in
  // flight where the paths meet): the last blocks ask again for the last block, which costs their turns in the memory pipeline
  // and nothing else.
  auto step = [&](int k, auto SS, Regs& cur) {
    constexpr int s = decltype(SS)::value;
    const int kn = blk(min(k + 1, NB - 1));
    // the mix of this wave's four ranks: operand B = Y_r(j = 4 g .. 4 g + 3, m = n), gathered from the four rows of its lane
    u32x2 yv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) yv[t] = *reinterpret_cast<const u32x2*>(&y_s[((4 * g + t) * 16 + n) * MU_LDY + rk + 8 * s]);
    f32x4 d[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
      const u32x2 yb = {__builtin_amdgcn_perm(yv[1][q >> 1], yv[0][q >> 1], sel), __builtin_amdgcn_perm(yv[3][q >> 1], yv[2][q >> 1], sel)};
      d[q] = YmDot<T>::mfma16(u32x2{cur.s[q >> 1][2 * (q & 1)], cur.s[q >> 1][2 * (q & 1) + 1]}, yb, f32x4{0.f, 0.f, 0.f, 0.f});
    }
    load_s(cur, kn, s);
    // d[q][t] = Z_r(i = 4 g + t, m = n) of slot 4 wv + q
#pragma unroll
    for (int t = 0; t < 4; ++t)
      *reinterpret_cast<u32x2*>(&z_s[s][((4 * g + t) * 16 + n) * MU_LDZ + 4 * wv]) = u32x2{ym_pack<T>(d[0][t], d[1][t]), ym_pack<T>(d[2][t], d[3][t])};
    mu_barrier();                                   // Z of the step is whole (the other step's buffer was last read a barrier ago)
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      const u32x4 zv = *reinterpret_cast<const u32x4*>(&z_s[s][((2 * wv + ii) * 16 + n) * MU_LDZ + 8 * g]);
#pragma unroll
      for (int nt = 0; nt < NTQ; ++nt) acc[ii][nt] = YmDot<T>::mfma(cur.u[ii][nt], zv, acc[ii][nt]);
    }
    load_u(cur, kn, s);
  };
  using S0 = std::integral_constant<int, 0>; using S1 = std::integral_constant<int, 1>;
  Regs ra, rb;
  // Block k asks for Y of block k + 2 into the registers `yl` that block k gave to LDS, and puts block k + 1 from `ys` into LDS at
  // its end.  (Loads return to a wave in the order it asked, and S and U are asked for one block ahead, so Y in effect has one
  // block's time as well; what bounds a step is the 112 KB per workgroup that 256 workgroups draw from L2 and memory, about
  // 1.4 us against 0.5 us for a step without loads.)
  auto block = [&](int k, u32x4 (&yl)[4], const u32x4 (&ys)[4]) {
    load_y(yl, blk(min(k + 2, NB - 1)));
    step(k, S0{}, ra);
    step(k, S1{}, rb);
    store_y(ys);                                    // every wave is past the barrier of the step: nobody reads this block of Y any more
    mu_barrier();                                   // Y of the next block is whole
  };

  u32x4 y0[4], y1[4];
  load_y(y0, blk(0)); load_s(ra, blk(0), 0); load_u(ra, blk(0), 0); load_s(rb, blk(0), 1); load_u(rb, blk(0), 1);
  load_y(y1, blk(min(1, NB - 1)));
  store_y(y0);
  mu_barrier();
  TR6(1);
  int k = 0;
  for (; k + 1 < NB; k += 2) {
    block(k, y0, y1);
    block(k + 1, y1, y0);
    TR6(2 + ((k >> 1) & 7));
  }
  if (k < NB) block(k, y0, y1);
  TR6(14);

  // acc[ii][nt][t] = out(m = m0 + n, column (2 wv + ii) Q + 16 nt + 4 g + t).  The tile (16 rows x 16 Q columns) goes through LDS
  // (over Y and the first Z buffer, which nobody reads any more: every wave is past the last step's barrier) so that it leaves
  // in whole rows: 16 bytes per lane, neighbouring lanes on neighbouring columns.
  using V4 = typename TypeTraits<T>::vec4;
  using V8 = typename TypeTraits<T>::vec8;
  const int OLD = 16 * Q + 8;
  uint16_t* const o_s = mu_lds;
#pragma unroll
  for (int ii = 0; ii < 2; ++ii)
#pragma unroll
    for (int nt = 0; nt < NTQ; ++nt) {
      const int q = 16 * nt + 4 * g;
      if (q < Q) {
        V4 o;
#pragma unroll
        for (int t = 0; t < 4; ++t) o[t] = TypeTraits<T>::from_f32(acc[ii][nt][t]);
        *reinterpret_cast<V4*>(&o_s[n * OLD + (2 * wv + ii) * Q + q]) = o;
      }
    }
  mu_barrier();
  const int ppr = 2 * Q;                                   // 16-byte pieces per row
  for (int pi = tid; pi < 16 * ppr; pi += MU_NT) {
    const int mr = pi / ppr, col = (pi - mr * ppr) * 8, m = m0 + mr;
    if (m >= M) break;
    const V8 rv8 = *reinterpret_cast<const V8*>(&o_s[mr * OLD + col]);
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = TypeTraits<T>::to_f32(rv8[e]);
    if (p.bias) {
      const V8 bv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.bias) + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += TypeTraits<T>::to_f32(bv[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = apply_act(v[e], p.act);
    if (p.gate || p.resid) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = TypeTraits<T>::to_f32(TypeTraits<T>::from_f32(v[e]));
      if (p.gate) {
        const V8 gv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.gate) + (int64_t)(m / p.gate_rows) * p.ld_gate + col);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= TypeTraits<T>::to_f32(gv[e]);
      }
      if (p.resid) {
        const V8 rv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.resid) + (int64_t)m * p.ld_resid + col);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += TypeTraits<T>::to_f32(rv[e]);
      }
    }
    V8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32(v[e]);
    *reinterpret_cast<V8*>(reinterpret_cast<T*>(p.out) + (int64_t)m * p.ldo + col) = o;
  }
  TR6(15);
}

// The re-laying of U and S (side_prep_item) as a launch of its own: one thread per piece.
template <typename T>
__global__ __launch_bounds__(256) void mixu_prep_kernel(SidePrep s) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < s.items) side_prep_item<T>(s, idx);
}

namespace {
template <typename T>
void* mixu_fn(int ntq) {
  switch (ntq) {
    case 1: return (void*)blast_mixu_kernel<T, 1>;
    case 2: return (void*)blast_mixu_kernel<T, 2>;
    case 3: return (void*)blast_mixu_kernel<T, 3>;
    case 4: return (void*)blast_mixu_kernel<T, 4>;
    case 5: return (void*)blast_mixu_kernel<T, 5>;
    default: return nullptr;
  }
}
}  // namespace

bool blast_mixu_plan(const void* Y, const void* S, const void* U, const void* out, int64_t ldo, const GemmArgs& ep, int M, int b, int R, int Q,
                     int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype, void* scratch, size_t scratch_bytes, SidePrep* job, bool u_rq) {
  if (dtype != BLR_F16 && dtype != BLR_BF16) return false;
  if (b != 16 || Q % 8 || Q > 80 || Q < 8 || R % 32 || M < 1) return false;
  if (!aligned(Y, 16) || !aligned(U, 16) || !aligned(out, 16) || ldo % 8) return false;
  if ((ep.bias && !aligned(ep.bias, 16)) || (ep.gate && (!aligned(ep.gate, 16) || ep.ld_gate % 8 || ep.gate_rows < 1)) ||
      (ep.resid && (!aligned(ep.resid, 16) || ep.ld_resid % 8))) return false;
  const int64_t y_bytes = (int64_t)b * M * R * 2;
  if (y_bytes >= (int64_t)YM_OOB || (int64_t)b * Q * R * 2 >= (int64_t)YM_OOB || (int64_t)b * b * R * 2 >= (int64_t)YM_OOB) return false;
  if (cdiv(M, MU_BM) >= 2147483647LL) return false;
  if (!(dtype == BLR_F16 ? mixu_fn<f16>((int)cdiv(Q, 16)) : mixu_fn<bf16>((int)cdiv(Q, 16)))) return false;
  const size_t ut_bytes = align_up((size_t)b * Q * R * 2, 256), sp_bytes = (size_t)b * b * R * 2;
  if (!scratch || scratch_bytes < ut_bytes + sp_bytes || !aligned(scratch, 16)) return false;
  if (job) {
    job->U = U; job->S = S; job->Ut = scratch; job->Sp = reinterpret_cast<char*>(scratch) + ut_bytes;
    job->Q = Q; job->R = R; job->u_rq = u_rq ? 1 : 0; job->s_si = s_si; job->s_sj = s_sj; job->s_sr = s_sr;
    job->items = (int64_t)b * (R / 8) * Q + (int64_t)R * 64;
  }
  return true;
}

// out (M, b Q) = [mix(S, Y)_i U_i]_i with the fused output stage of `ep` (bias, act, gate, resid; its other members are not
// read).  Y (b, M, R), U (b, Q, R) of dtype.  scratch: room for U and S re-laid (b Q R + b b R elements, rounded up to 256
// bytes each); prepared: an earlier launch of the call has already put them there.  Returns BLR_OK, a negative blr_status, or 1
// when the shape is not for this kernel (b other than 16, blocks wider than 80 columns or not a multiple of 8, rank not a
// multiple of 32, unaligned operands, fp32).
int blast_mixu_launch(const void* Y, const void* S, const void* U, void* out, int64_t ldo, const GemmArgs& ep, int M, int b, int R, int Q,
                      int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                      hipStream_t st, bool prepared, bool u_rq) {
  (void)s_layout;
  SidePrep job = {};
  if (!blast_mixu_plan(Y, S, U, out, ldo, ep, M, b, R, Q, s_si, s_sj, s_sr, dtype, scratch, scratch_bytes, &job, u_rq)) return 1;
  void* fn = dtype == BLR_F16 ? mixu_fn<f16>((int)cdiv(Q, 16)) : mixu_fn<bf16>((int)cdiv(Q, 16));
  MixuParams p = {};
  p.Y = Y; p.out = out; p.ldo = ldo; p.M = M; p.R = R; p.Q = Q; p.y_bytes = (uint32_t)((int64_t)b * M * R * 2);
  p.bias = ep.bias; p.act = ep.act; p.gate = ep.gate; p.gate_rows = ep.gate ? ep.gate_rows : 1; p.ld_gate = ep.ld_gate;
  p.resid = ep.resid; p.ld_resid = ep.ld_resid;
  p.Ut = job.Ut; p.Sp = job.Sp;
  p.rotate = 1;
  if (!prepared) {
    const unsigned tg = (unsigned)cdiv(job.items, 256);
    if (dtype == BLR_F16) hipLaunchKernelGGL(mixu_prep_kernel<f16>, dim3(tg), dim3(256), 0, st, job);
    else hipLaunchKernelGGL(mixu_prep_kernel<bf16>, dim3(tg), dim3(256), 0, st, job);
    BLR_CHECK_LAUNCH("mixu_prep");
  }
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3((unsigned)cdiv(M, MU_BM)), dim3(MU_NT), args, 0, st);
  if (e != hipSuccess) { set_error("blast_mixu: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

// ---- narrow input AND output blocks: the whole call in one launch, neither Y nor Z in memory ------------------------------
//
// With input blocks of at most 96 columns the chunk of V that a step of blast_mixu_kernel's walk over the rank needs (16 input
// blocks x P x 32 ranks) is as small as its chunk of U, so the workgroup forms the step's Y itself instead of reading it: wave w
// keeps its rows of x for input blocks 2 w and 2 w + 1 in registers (operand B, 16 rows x P), loads the 32 ranks of V_2w and
// V_2w+1 (operand A: V re-laid like U, rank-major with k contiguous, in the order the lanes read it, k padded to 32 KS with
// zeros) and leaves Y^T (ranks x rows) as T in LDS - four consecutive ranks per lane.  The rest of the step is the step of
// blast_mixu_kernel: mix of four ranks per wave into Z (LDS), barrier, products with U_2w, U_2w+1 into the 16 x 16 Q results
// that stay in registers for the whole call.  Three barriers per step; Y and Z have one buffer each (every reader of a buffer is
// past the barrier that precedes its next writer in program order).
struct OneParams {
  const void* x; int64_t ldx; uint32_t x_bytes;
  const void* Vp; const void* Sp; const void* Ut; void* out; int64_t ldo;     // Vp (step, j, half, kstep, lane, 8), Sp, Ut as for blast_mixu_kernel
  int M, P, R, Q;
  const void* bias; int act;
  const void* gate; int gate_rows; int64_t ld_gate;
  const void* resid; int64_t ld_resid;
};

template <typename T, int NTQ, int KS>
__global__ __launch_bounds__(MU_NT) void blast_one_kernel(OneParams p) {
  constexpr int LDY = 40;                                    // two-byte elements per LDS row of Y and Z (32 ranks / slots + 8)
  constexpr int OSN = 16 * (16 * 80 + 8);                      // the tile on its way out: 16 rows of up to 16 x 80 columns (+ 8)
  __shared__ __attribute__((aligned(16))) uint16_t one_lds[2 * 256 * LDY > OSN ? 2 * 256 * LDY : OSN];
  uint16_t* const y_s = one_lds;                             // [input block j][row m][rank of the step]
  uint16_t* const z_s = one_lds + 256 * LDY;                 // [output block i][row m][slot]
  const int tid = threadIdx.x, wv = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
  const int M = p.M, P = p.P, R = p.R, Q = p.Q;
  const int m0 = (int)blockIdx.x * MU_BM;
  const int NSTEP = R / 32;
  const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.x), 0, p.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t vbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Vp), 0, (uint32_t)((int64_t)NSTEP * 16 * 2 * KS * 1024), 0x00020000);
  const __amdgpu_buffer_rsrc_t sbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Sp), 0, (uint32_t)(256 * R * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t ubuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.Ut), 0, (uint32_t)((int64_t)16 * Q * R * 2), 0x00020000);
  // the rows of x: operand B of the first products, lane (n, g) = row m0 + n, k = 32 ks + 8 g .. + 7 of input block 2 wv + jj
  u32x4 xr[2][KS];
#pragma unroll
  for (int jj = 0; jj < 2; ++jj)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int k = 32 * ks + 8 * g;
      const uint32_t off = (m0 + n < M && k < P) ? (uint32_t)((int64_t)(m0 + n) * p.ldx + (int64_t)(2 * wv + jj) * P + k) * 2u : YM_OOB;
      xr[jj][ks] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xbuf, off, 0, 0));
    }
  const uint32_t voff = (uint32_t)((2 * wv) * 2 * KS * 1024 + l * 16);     // + ((jj 2 + nt) KS + ks) 1024; a step is 16 * 2 * KS KiB further
  const uint32_t soff = (uint32_t)((2 * wv) * 64 + l) * 16u;
  const uint32_t uoff = (uint32_t)(((int64_t)(2 * wv) * (R / 8) + g) * Q + n) * 16u;
  const uint32_t uoff_last = 16 * (NTQ - 1) + n < Q ? uoff : YM_OOB;
  const uint32_t uis = (uint32_t)((R / 8) * Q) * 16u;
  struct Regs { u32x4 s[2]; u32x4 u[2][NTQ]; };
  u32x4 vr[2][2][KS];
  auto load_v = [&](int s) {
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          vr[jj][nt][ks] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(vbuf, voff + (uint32_t)(((jj * 2 + nt) * KS + ks) * 1024), (uint32_t)s * (uint32_t)(16 * 2 * KS * 1024), 0));
  };
  auto load_s = [&](Regs& r, int s) {                        // ranks 32 s + 4 wv + q
#pragma unroll
    for (int q = 0; q < 2; ++q) r.s[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(sbuf, soff + (uint32_t)q * 1024u, (uint32_t)(32 * s) * 512u, 0));
  };
  auto load_u = [&](Regs& r, int s) {
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
      for (int nt = 0; nt < NTQ; ++nt)
        r.u[ii][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ubuf, (nt == NTQ - 1 ? uoff_last : uoff) + (uint32_t)nt * 256u,
                                                                                        (uint32_t)(4 * s * Q) * 16u + (uint32_t)ii * uis, 0));
  };
  f32x4 acc[2][NTQ];
#pragma unroll
  for (int ii = 0; ii < 2; ++ii)
#pragma unroll
    for (int nt = 0; nt < NTQ; ++nt) acc[ii][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // Workgroups start at different steps (the fp32 sums keep a fixed order per row tile): they would otherwise all ask the L2s
  // for the same lines of V, U and S at the same moment.
  const int rot = (int)(blockIdx.x % (unsigned)NSTEP);
  auto stp = [&](int s) { const int v = s + rot; return v >= NSTEP ? v - NSTEP : v; };

  // No load sits under a condition (the compiler would then wait for everything in flight where the paths meet): the last steps
  // ask again for the last step, which costs their turns in the memory pipeline and nothing else.
  auto step = [&](int s, Regs& cur) {
    const int s1 = stp(min(s + 1, NSTEP - 1)), s2 = stp(min(s + 2, NSTEP - 1));
    // Y^T of the step: ranks 16 nt + 4 g + t of rows m = n, input blocks 2 wv and 2 wv + 1
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) y = YmDot<T>::mfma(vr[jj][nt][ks], xr[jj][ks], y);
        *reinterpret_cast<u32x2*>(&y_s[((2 * wv + jj) * 16 + n) * LDY + 16 * nt + 4 * g]) = u32x2{ym_pack<T>(y[0], y[1]), ym_pack<T>(y[2], y[3])};
      }
    load_v(s1);
    mu_barrier();                                   // Y of the step is whole
    // the mix of this wave's four ranks: operand B = Y_r(j = 4 g .. 4 g + 3, m = n), gathered from the four rows of its lane
    u32x2 yv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) yv[t] = *reinterpret_cast<const u32x2*>(&y_s[((4 * g + t) * 16 + n) * LDY + 4 * wv]);
    f32x4 d[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
      const u32x2 yb = {__builtin_amdgcn_perm(yv[1][q >> 1], yv[0][q >> 1], sel), __builtin_amdgcn_perm(yv[3][q >> 1], yv[2][q >> 1], sel)};
      d[q] = YmDot<T>::mfma16(u32x2{cur.s[q >> 1][2 * (q & 1)], cur.s[q >> 1][2 * (q & 1) + 1]}, yb, f32x4{0.f, 0.f, 0.f, 0.f});
    }
    load_s(cur, s2);
#pragma unroll
    for (int t = 0; t < 4; ++t)
      *reinterpret_cast<u32x2*>(&z_s[((4 * g + t) * 16 + n) * LDY + 4 * wv]) = u32x2{ym_pack<T>(d[0][t], d[1][t]), ym_pack<T>(d[2][t], d[3][t])};
    mu_barrier();                                   // Z of the step is whole; nobody reads this step's Y any more
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      const u32x4 zv = *reinterpret_cast<const u32x4*>(&z_s[((2 * wv + ii) * 16 + n) * LDY + 8 * g]);
#pragma unroll
      for (int nt = 0; nt < NTQ; ++nt) acc[ii][nt] = YmDot<T>::mfma(cur.u[ii][nt], zv, acc[ii][nt]);
    }
    load_u(cur, s2);
  };
  Regs ra, rb;
  load_v(stp(0));
  load_s(ra, stp(0)); load_u(ra, stp(0));
  load_s(rb, stp(min(1, NSTEP - 1))); load_u(rb, stp(min(1, NSTEP - 1)));
  int s = 0;
  for (; s + 1 < NSTEP; s += 2) { step(s, ra); step(s + 1, rb); }
  if (s < NSTEP) step(s, ra);
  mu_barrier();                                     // every wave is through with Z: the tile may go over it

  // the tile (16 rows x 16 Q columns) leaves through LDS in whole rows, as in blast_mixu_kernel
  using V4 = typename TypeTraits<T>::vec4;
  using V8 = typename TypeTraits<T>::vec8;
  const int OLD = 16 * Q + 8;
  uint16_t* const o_s = one_lds;
#pragma unroll
  for (int ii = 0; ii < 2; ++ii)
#pragma unroll
    for (int nt = 0; nt < NTQ; ++nt) {
      const int q = 16 * nt + 4 * g;
      if (q < Q) {
        V4 o;
#pragma unroll
        for (int t = 0; t < 4; ++t) o[t] = TypeTraits<T>::from_f32(acc[ii][nt][t]);
        *reinterpret_cast<V4*>(&o_s[n * OLD + (2 * wv + ii) * Q + q]) = o;
      }
    }
  mu_barrier();
  const int ppr = 2 * Q;
  for (int pi = tid; pi < 16 * ppr; pi += MU_NT) {
    const int mr = pi / ppr, col = (pi - mr * ppr) * 8, m = m0 + mr;
    if (m >= M) break;
    const V8 rv8 = *reinterpret_cast<const V8*>(&o_s[mr * OLD + col]);
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = TypeTraits<T>::to_f32(rv8[e]);
    if (p.bias) {
      const V8 bv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.bias) + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += TypeTraits<T>::to_f32(bv[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = apply_act(v[e], p.act);
    if (p.gate || p.resid) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = TypeTraits<T>::to_f32(TypeTraits<T>::from_f32(v[e]));
      if (p.gate) {
        const V8 gv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.gate) + (int64_t)(m / p.gate_rows) * p.ld_gate + col);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= TypeTraits<T>::to_f32(gv[e]);
      }
      if (p.resid) {
        const V8 rv = *reinterpret_cast<const V8*>(reinterpret_cast<const T*>(p.resid) + (int64_t)m * p.ld_resid + col);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += TypeTraits<T>::to_f32(rv[e]);
      }
    }
    V8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32(v[e]);
    *reinterpret_cast<V8*>(reinterpret_cast<T*>(p.out) + (int64_t)m * p.ldo + col) = o;
  }
}

// V (16, P, R) -> Vp (step, j, half of the step's ranks, k step, lane (n, g), 8): element e of lane (n, g) is
// V_j[32 ks + 8 g + e][32 step + 16 half + n], zero past P; then U and S as side_prep_item lays them.  One thread per 16-byte piece.
template <typename T>
__global__ __launch_bounds__(256) void one_prep_kernel(const T* __restrict__ V, T* __restrict__ Vp, int P, int KS, SidePrep s) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nv = (int64_t)(s.R / 32) * 16 * 2 * KS * 64;
  if (idx < nv) {
    const int l = (int)(idx & 63), n = l & 15, g = l >> 4;
    int64_t c = idx >> 6;
    const int ks = (int)(c % KS); c /= KS;
    const int half = (int)(c & 1); c >>= 1;
    const int j = (int)(c & 15), step = (int)(c >> 4);
    typename TypeTraits<T>::vec8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = 32 * ks + 8 * g + e;
      o[e] = k < P ? V[((int64_t)j * P + k) * s.R + 32 * step + 16 * half + n] : (T)0.0f;
    }
    *reinterpret_cast<typename TypeTraits<T>::vec8*>(Vp + idx * 8) = o;
  } else if (idx - nv < s.items) {
    side_prep_item<T>(s, idx - nv);
  }
}

namespace {
template <typename T, int KS>
void* one_fn_ks(int Q) {
  return Q <= 48 ? (void*)blast_one_kernel<T, 3, KS> : (void*)blast_one_kernel<T, 5, KS>;
}
template <typename T>
void* one_fn(int Q, int ks) {
  switch (ks) {
    case 1: return one_fn_ks<T, 1>(Q);
    case 2: return one_fn_ks<T, 2>(Q);
    case 3: return one_fn_ks<T, 3>(Q);
    default: return nullptr;
  }
}
}  // namespace

// out = BLAST(x) for 16 input blocks of at most 96 columns and 16 output blocks of at most 80, U (b, Q, R) or (u_rq) (b, R, Q): one launch after the
// re-laying of V, U and S into scratch (b (32 ceil(P / 32) + Q + b) R elements, each part rounded up to 256 bytes).  The fused
// output stage is taken from `ep`.  Returns BLR_OK, a negative blr_status, or 1 when the shape is not for this kernel.
int blast_one_launch(const void* x, int64_t ldx, const void* U, const void* V, const void* S, void* out, int64_t ldo, const GemmArgs& ep,
                     int M, int in_f, int b, int R, int Q, int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype,
                     void* scratch, size_t scratch_bytes, hipStream_t st, bool u_rq) {
  if (dtype != BLR_F16 && dtype != BLR_BF16) return 1;
  if (b != 16 || in_f % 16) return 1;
  const int P = in_f / 16, KS = (int)cdiv(P, 32);
  if (P % 8 || P > 96 || Q % 8 || Q > 80 || Q < 8 || R % 32 || M < 1) return 1;
  if (!aligned(x, 16) || ldx % 8 || !aligned(U, 16) || !aligned(V, 16) || !aligned(out, 16) || ldo % 8) return 1;
  if ((ep.bias && !aligned(ep.bias, 16)) || (ep.gate && (!aligned(ep.gate, 16) || ep.ld_gate % 8 || ep.gate_rows < 1)) ||
      (ep.resid && (!aligned(ep.resid, 16) || ep.ld_resid % 8))) return 1;
  const int64_t x_elems = (int64_t)(M - 1) * ldx + in_f;
  if (x_elems * 2 >= (int64_t)YM_OOB || (int64_t)b * Q * R * 2 >= (int64_t)YM_OOB || (int64_t)b * b * R * 2 >= (int64_t)YM_OOB ||
      (int64_t)b * 32 * KS * R * 2 >= (int64_t)YM_OOB || cdiv(M, MU_BM) >= 2147483647LL) return 1;
  const size_t vp_bytes = align_up((size_t)b * 32 * KS * R * 2, 256), ut_bytes = align_up((size_t)b * Q * R * 2, 256), sp_bytes = (size_t)b * b * R * 2;
  if (!scratch || scratch_bytes < vp_bytes + ut_bytes + sp_bytes || !aligned(scratch, 16)) return 1;
  void* fn = dtype == BLR_F16 ? one_fn<f16>(Q, KS) : one_fn<bf16>(Q, KS);
  if (!fn) return 1;
  char* sp = reinterpret_cast<char*>(scratch);
  SidePrep job = {};
  job.U = U; job.S = S; job.Ut = sp + vp_bytes; job.Sp = sp + vp_bytes + ut_bytes;
  job.Q = Q; job.R = R; job.u_rq = u_rq ? 1 : 0; job.s_si = s_si; job.s_sj = s_sj; job.s_sr = s_sr;
  job.items = (int64_t)b * (R / 8) * Q + (int64_t)R * 64;
  {
    const int64_t nv = (int64_t)(R / 32) * 16 * 2 * KS * 64;
    const unsigned tg = (unsigned)cdiv(nv + job.items, 256);
    if (dtype == BLR_F16) hipLaunchKernelGGL(one_prep_kernel<f16>, dim3(tg), dim3(256), 0, st, (const f16*)V, (f16*)sp, P, KS, job);
    else hipLaunchKernelGGL(one_prep_kernel<bf16>, dim3(tg), dim3(256), 0, st, (const bf16*)V, (bf16*)sp, P, KS, job);
    BLR_CHECK_LAUNCH("one_prep");
  }
  OneParams p = {};
  p.x = x; p.ldx = ldx; p.x_bytes = (uint32_t)(x_elems * 2); p.Vp = sp; p.Sp = job.Sp; p.Ut = job.Ut; p.out = out; p.ldo = ldo;
  p.M = M; p.P = P; p.R = R; p.Q = Q;
  p.bias = ep.bias; p.act = ep.act; p.gate = ep.gate; p.gate_rows = ep.gate ? ep.gate_rows : 1; p.ld_gate = ep.ld_gate;
  p.resid = ep.resid; p.ld_resid = ep.ld_resid;
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3((unsigned)cdiv(M, MU_BM)), dim3(MU_NT), args, 0, st);
  if (e != hipSuccess) { set_error("blast_one: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace6(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace6), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

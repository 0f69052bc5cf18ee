// Two-stage BLAST decode kernel for a handful of token rows (M <= 4), U (b, r, q) / V (b, p, r).
//
// The whole call is one short dependency chain, so the kernel is built around latency rather
// than around phases:
//   * every workgroup that owns a slab of U starts by asking for (up to) all of it: up to 32
//     16-byte loads per lane go out before anything else is waited for, so HBM streams U while
//     stage 1 and the hand-over of its result are still in progress;
//   * there is no grid barrier.  Values that cross workgroups (stage-1 results y, split-k
//     partial outputs) are stored as 8-byte {fp32 bits, epoch} pairs with device-scope stores;
//     a consumer simply re-reads a pair until its tag equals the epoch of this call.  One store
//     and one load make up a hand-over, instead of store - wait - count - poll - load;
//   * the rank-space mix  z_i = sum_j S_ij * y_j  is a role of its own: a few of the first
//     workgroups each take a handful of r, fetch the tagged y of every j once, and publish z as
//     tagged pairs for the stage-2 slabs.
// The epoch lives in the workspace.  Every workgroup reads it when it starts and then checks
// in; the last one to check in advances it for the next call, which is safe because by then
// every workgroup of this call holds its own copy.  Tag 0 is never used, so a zero-filled
// workspace holds no valid pair.  Calls that share a workspace must be ordered on one stream.
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include "blr_common.h"
#include "blr_decode.h"
#include "blr_decode_dev.h"

namespace blr {

namespace {
// 16-byte loads of the U slab held in registers per lane (fewer when the accumulators need the room)
constexpr int d2_pf(int MT, int WB = 16) { return MT * (128 / WB) >= 64 ? 16 : (MT <= 1 ? 32 : (MT <= 2 ? 24 : 16)); }
#ifndef BLR_D2_FIRST
#define BLR_D2_FIRST 8
#endif
constexpr int D2_FIRST = BLR_D2_FIRST;   // loads of the U slab that go out right behind the V loads of stage 1
constexpr int D2_UNR = 8;             // loads in flight per lane while streaming the rest of a slab
constexpr int d2_unr1(int) { return 8; }   // loads in flight per lane in stage 1
constexpr int d2_ks1_max(int MT) { return MT <= 2 ? 8 : 4; } // most k-slices of stage 1 (the mix fetches them all at once)
constexpr int D2_AS = 4096;           // fp32 activations staged in LDS (MT * k-chunk <= this)
constexpr int D2_NC_MAX = 512;
}  // namespace

#ifdef BLR_TRACE
__device__ unsigned long long g_trace2[1024 * 16];
#define TR2(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) g_trace2[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR2(i) do {} while (0)
#endif

struct Decode2Params {
  const void* x; int64_t ldx;
  const void* V; const void* U; const void* S;
  const f16* u_scales; const f16* v_scales;      // quantized weights only
  void* out; int64_t ldo;
  int u_nk, rpw, kl_log2;                        // U (bo, q, r): rows of U per wave, log2 of the 16-byte loads per row and lane
  int perm_per; int64_t o_bs, o_ns;              // Monarch permutation period; output strides of (block, column)
  int zrep;                                      // bo == 1: z is published in zrep copies so that the slabs do not all poll one address range
  int M, b, bo, P, R, Q;                         // b blocks of the input (stage 1), bo blocks of the output (stage 2)
  int64_t s_si, s_sj, s_sr;
  int lpr1_log2, nch1, ks1, kc1, items1;
  int lpr2_log2, nch2, ks2, kc2, items2, pfn, kpad2;
  int itemsM, rch_log2, pf_depth, pf_first, x_vec;
  unsigned long long* ypart;           // [ks1][b][M][R] tagged
  unsigned long long* zt;              // [b][M][R] tagged
  unsigned long long* opart;           // [ks2 - 1][b][M][Q] tagged
  unsigned* epoch_word; unsigned* arrive_word; unsigned* err_word;
  unsigned spin_limit;
};

// Sum of the row slots of a wave, then of the four waves; thread `col` < NC ends up with the
// total of column `col` for each of the MT rows (returned through `tot`, valid for tid < NC).
template <int MT, int EPL>
__device__ __forceinline__ void wg_reduce(float (&acc)[MT][EPL], int lpr, int cv, float* red, int NC, float (&tot)[MT][2]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int o = lpr; o < 64; o <<= 1) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[m][e] += __shfl_xor(acc[m][e], o, 64);
  }
  __syncthreads();
  if (lane < lpr) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int e = 0; e < EPL; ++e) red[(wave * MT + m) * D2_NC_MAX + cv * EPL + e] = acc[m][e];
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int col = tid + h * 256;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      float v = 0.0f;
      if (col < NC)
        v = red[(0 * MT + m) * D2_NC_MAX + col] + red[(1 * MT + m) * D2_NC_MAX + col] +
            red[(2 * MT + m) * D2_NC_MAX + col] + red[(3 * MT + m) * D2_NC_MAX + col];
      tot[m][h] = v;
    }
  }
}

template <typename T, int MT, int WB>
__global__ __launch_bounds__(256, 2) void decode2_kernel(Decode2Params p) {
  constexpr int EPL = 128 / WB;                      // weights per 16-byte load
  constexpr int D2_PF = d2_pf(MT, WB);
  constexpr int D2_UNR1 = d2_unr1(MT);
  constexpr int D2_KS1_MAX = d2_ks1_max(MT);
  __shared__ float a_s[D2_AS];
  __shared__ float red[4 * MT * D2_NC_MAX];
  constexpr int KLD = D2_AS / MT;
  const int tid = threadIdx.x;
  const int w = blockIdx.x, G = gridDim.x;
  const int M = p.M;
  const unsigned long long t_begin = wall_clock64();

  TR2(0);
  // ---- epoch of this call ------------------------------------------------------------------
  // (a plain, cached load: the word was last written before this kernel began, and hundreds of workgroups asking one
  // address for a device-scope copy would queue up at a single memory channel - with every later load of theirs behind it)
  unsigned epoch = *reinterpret_cast<const volatile unsigned*>(p.epoch_word) + 1u;
  if (epoch == 0u) epoch = 1u;

  // ---- stage-2 slab of this workgroup --------------------------------------------------------
  const int item2 = G - 1 - w;
  const bool has2 = item2 < p.items2;
  const int lpr2 = 1 << p.lpr2_log2, rpp2 = 256 >> p.lpr2_log2;
  const int cv2 = tid & (lpr2 - 1), rs2 = tid >> p.lpr2_log2;
  const int nc2 = has2 ? item2 % p.nch2 : 0;
  const int t2 = has2 ? item2 / p.nch2 : 0;
  const int i2 = t2 % p.bo, ksi2 = t2 / p.bo;
  const int zi = p.zrep > 1 ? nc2 % p.zrep : i2;     // which published copy of z this slab reads
  const int k0_2 = ksi2 * p.kc2;
  const int kcur2 = min(p.kc2, p.R - k0_2);
  const int NC2 = lpr2 * EPL;
  const int n0_2 = nc2 * NC2;
  const int n2 = n0_2 + cv2 * EPL;
  const bool col_ok2 = n2 < p.Q;
  const __amdgpu_buffer_rsrc_t ubuf = wbuf(p.U, (uint32_t)((int64_t)p.bo * p.R * p.Q * WB / 8));
  // U (bo, q, r) ("NK", two-byte weights only): a wave owns rpw consecutive rows of U_i, a lane 8 consecutive k
  // of every 512; load u of a lane is row u >> kl_log2, piece u & (KL - 1).  No k-split, no partial sums.
  const int nk_row0 = nc2 * 4 * p.rpw + (tid >> 6) * p.rpw;
  const uint32_t uoff = p.u_nk ? (uint32_t)((((int64_t)i2 * p.Q + nk_row0) * p.R + (tid & 63) * 8) * 2)
                               : (uint32_t)((((int64_t)i2 * p.R + k0_2 + rs2) * p.Q + (col_ok2 ? n2 : 0)) * WB / 8);   // bytes, first load of this lane
  const uint32_t ustep = (uint32_t)((int64_t)rpp2 * p.Q * WB / 8);                                            // bytes between a lane's loads
  auto u_soff = [&](int u) -> uint32_t {
    return p.u_nk ? (uint32_t)(((u >> p.kl_log2) * p.R + (u & ((1 << p.kl_log2) - 1)) * 512) * 2) : (uint32_t)u * ustep;
  };

  u32x4 pf[D2_PF];                                   // only slots below pfn are ever read after the prefetch
  auto issue_prefetch = [&](int lo, int hi) {        // loads lo .. hi - 1 of the slab (hi is cut at pfn)
#pragma unroll
    for (int u = 0; u < D2_PF; ++u) {
      if (u >= lo && u < hi && u < p.pfn) {
        // pacing: at most pf_depth of this lane's loads in flight, so that the queues of the memory
        // system stay short enough for the small hand-over accesses of other workgroups to get through
        if (u >= D2_FIRST) {
          if (u >= 2 && p.pf_depth == 2) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
          else if (u >= 3 && p.pf_depth == 3) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
          else if (u >= 4 && p.pf_depth == 4) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
          else if (u >= 6 && p.pf_depth == 6) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
          else if (u >= 8 && p.pf_depth == 8) asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
          else if (u >= 12 && p.pf_depth == 12) asm volatile("s_waitcnt vmcnt(11)" ::: "memory");
          else if (u >= 16 && p.pf_depth == 16) asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        }
        pf[u] = ldw16(ubuf, uoff, u_soff(u));
      }
    }
  };
  int pf_lo = 0;                                       // loads of the slab already asked for

  // Mix role (the first workgroups): its S values depend on nothing, so they are asked for first.
  // S(i = g, j = u, r) for this thread's (g, r); indices are clamped so that every load is legal.
  float sv[16];
  if (w < p.itemsM) {
    const int g = min(tid >> p.rch_log2, p.bo - 1);   // (replicas of a single output block all use S of block 0)
    const int r = min(w * (1 << p.rch_log2) + (tid & ((1 << p.rch_log2) - 1)), p.R - 1);
    const T* Sp = reinterpret_cast<const T*>(p.S);
    if (Sp) {                                           // one uniform branch, then unconditional loads
#pragma unroll
      for (int u = 0; u < 16; ++u)
        sv[u] = TypeTraits<T>::to_f32(Sp[(int64_t)g * p.s_si + (int64_t)min(u, p.b - 1) * p.s_sj + (int64_t)r * p.s_sr]);
    } else {
#pragma unroll
      for (int u = 0; u < 16; ++u) sv[u] = 1.0f;
    }
  }

  // Check-in: once the epoch has arrived this workgroup counts itself (no value comes back, so nothing
  // waits on it).  Workgroup 0 advances the epoch word at its very end, after seeing every check-in.
  auto check_in = [&]() {
    if (tid == 0) {
      asm volatile("" ::"v"(epoch) : "memory");
      (void)__hip_atomic_fetch_add(&p.arrive_word[(w % D2_SHARDS) * 64], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  // ---- stage 1: y[ks][j][m][n] = sum_k x[m, j P + k] V_j[k, n] over this workgroup's k-slice ----
  if (w < p.items1) {
    const int lpr1 = 1 << p.lpr1_log2, rpp1 = 256 >> p.lpr1_log2;
    const int cv1 = tid & (lpr1 - 1), rs1 = tid >> p.lpr1_log2;
    const int nc1 = w % p.nch1;
    const int t1 = w / p.nch1;
    const int j = t1 % p.b, ks = t1 / p.b;
    const int k0 = ks * p.kc1, kc = min(p.kc1, p.P - k0);
    const int NC1 = lpr1 * EPL;
    const int n0 = nc1 * NC1, n = n0 + cv1 * EPL;
    const bool col_ok = n < p.R;
    const __amdgpu_buffer_rsrc_t vbuf = wbuf(p.V, (uint32_t)((int64_t)p.b * p.P * p.R * WB / 8));
    const uint32_t voff = (uint32_t)((((int64_t)j * p.P + k0 + rs1) * p.R + (col_ok ? n : 0)) * WB / 8);
    const uint32_t vstep = (uint32_t)((int64_t)rpp1 * p.R * WB / 8);

    // Batches are always full: rows past the end of the slice meet a zero activation.
    const int nbatch = ((kc + rpp1 - 1) / rpp1 + D2_UNR1 - 1) / D2_UNR1;
    const int kpad = nbatch * D2_UNR1 * rpp1;          // rows the batches touch (the host keeps this within KLD)
    // The activations go first of all (loads come back in order, and they are needed first).
    const T* xp = reinterpret_cast<const T*>(p.x);
    constexpr int XR = 4;
    T xr[XR];
#pragma unroll
    for (int q = 0; q < XR; ++q) {
      const int idx = tid + q * 256;
      const int m = min(idx / kpad, M - 1), ka = min(idx % kpad, kc - 1);
      xr[q] = xp[(int64_t)m * p.ldx + (int64_t)j * p.P + k0 + ka];
    }
    u32x4 raw[D2_UNR1];
#pragma unroll
    for (int u = 0; u < D2_UNR1; ++u) raw[u] = ldw16(vbuf, voff, (uint32_t)u * vstep);
    // The first loads of this workgroup's slab of U go out right behind: what heads the dependency chain is asked
    // for first by every workgroup and comes back first (loads return in order), and the U stream is under way
    // while stage 1 is being computed and handed over.
    // (Straight-line, unconditional loads: a slot this workgroup does not have gets an offset beyond the buffer, which
    // reads as zero without touching memory - so the compiler knows how many loads follow the V loads and waits
    // for exactly those.)
#pragma unroll
    for (int u = 0; u < D2_FIRST; ++u) pf[u] = ldw16(ubuf, (has2 && u < p.pfn) ? uoff : 0x80000000u, u_soff(u));
    pf_lo = D2_FIRST;
#pragma unroll
    for (int q = 0; q < XR; ++q) {
      const int idx = tid + q * 256;
      if (idx < MT * kpad) {
        const int m = idx / kpad, ka = idx - m * kpad;
        a_s[m * KLD + ka] = (m < M && ka < kc) ? TypeTraits<T>::to_f32(xr[q]) : 0.0f;
      }
    }
    for (int idx = tid + XR * 256; idx < MT * kpad; idx += 256) {   // long slices only
      const int m = idx / kpad, ka = idx - m * kpad;
      a_s[m * KLD + ka] = (m < M && ka < kc) ? TypeTraits<T>::to_f32(xp[(int64_t)m * p.ldx + (int64_t)j * p.P + k0 + ka]) : 0.0f;
    }
    check_in();
    __syncthreads();

    float acc[MT][EPL];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
    for (int bi = 0; bi < nbatch; ++bi) {
#pragma unroll
      for (int u = 0; u < D2_UNR1; ++u) {
        float wv[EPL];
        cvtw<T, WB>(raw[u], wv);
        const int k = rs1 + (bi * D2_UNR1 + u) * rpp1;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float a = a_s[m * KLD + k];            // zero beyond the slice
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(a, wv[e], acc[m][e]);
        }
      }
      if (bi + 1 < nbatch) {                           // deeper slices than one batch (the planner avoids them)
#pragma unroll
        for (int u = 0; u < D2_UNR1; ++u)
          raw[u] = ldw16(vbuf, voff, (uint32_t)((bi + 1) * D2_UNR1 + u) * vstep);
      }
    }
    TR2(1);

    float tot[MT][2];
    wg_reduce<MT, EPL>(acc, lpr1, cv1, red, NC1, tot);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int col = tid + h * 256;
      if (col < NC1 && n0 + col < p.R) {
        const float vsc = (WB != 16) ? (float)p.v_scales[(int64_t)j * p.R + n0 + col] : 1.0f;   // per-rank scale of the codes of V
#pragma unroll
        for (int m = 0; m < MT; ++m)
          if (m < M) st_tag(&p.ypart[(((int64_t)ks * p.b + j) * M + m) * p.R + n0 + col], tot[m][h] * vsc, epoch);
      }
    }
    TR2(2);
  } else {
    check_in();
  }

  // ---- mix role: z[i][m][r] = sum_j S(i, j, r) * sum_ks y[ks][j][m][r] for RCH values of r, every i ------
  // Thread (g, rr): first g is the block column j whose y it fetches, then the block row i it emits.
  if (w < p.itemsM) {
    __syncthreads();                                   // the stage-1 use of a_s is over
    TR2(8);
    const int RCH = 1 << p.rch_log2;
    const int g = tid >> p.rch_log2, rr = tid & (RCH - 1);
    const int r = w * RCH + rr;
    // Monarch: the "mix" is a permutation - z[l][r] is the single value y[r / per][l * per + r % per]
    const bool perm = p.perm_per > 0;
    const int yj = perm ? r / p.perm_per : g;
    const int yr = perm ? g * p.perm_per + r % p.perm_per : r;
    const bool live = (perm ? g < p.bo : g < p.b) && r < p.R;          // fetches y of input block yj
    const bool live_o = g < (p.zrep > 1 ? p.zrep : p.bo) && r < p.R;   // emits z of output block (or replica) g
    const T* Sp = reinterpret_cast<const T*>(p.S);
    float ysum[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) ysum[m] = 0.0f;
    if (live) {
      unsigned long long yv[D2_KS1_MAX][MT];
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int ks = 0; ks < D2_KS1_MAX; ++ks) {
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            if (ks < p.ks1 && m < M) {
              yv[ks][m] = ld_tag(&p.ypart[(((int64_t)ks * p.b + yj) * M + m) * p.R + yr]);
              ok = ok && ((unsigned)(yv[ks][m] >> 32) == epoch);
            } else {
              yv[ks][m] = 0ull;
            }
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int ks = 0; ks < D2_KS1_MAX; ++ks)
#pragma unroll
        for (int m = 0; m < MT; ++m) ysum[m] += __uint_as_float((unsigned)yv[ks][m]);
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) a_s[m * 256 + tid] = ysum[m];     // [m][j][rr]
    __syncthreads();
    if (live_o) {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if (m < M) {
          float z = perm ? ysum[m] : 0.0f;
#pragma unroll
          for (int u = 0; u < 16; ++u) z = fmaf((u < p.b && !perm) ? sv[u] : 0.0f, a_s[m * 256 + min(u, p.b - 1) * RCH + rr], z);
          for (int j = 16; j < p.b && !perm; ++j)
            z = fmaf(Sp ? TypeTraits<T>::to_f32(Sp[(int64_t)min(g, p.bo - 1) * p.s_si + (int64_t)j * p.s_sj + (int64_t)r * p.s_sr]) : 1.0f, a_s[m * 256 + j * RCH + rr], z);
          st_tag(&p.zt[((int64_t)g * M + m) * p.R + r], z, epoch);
        }
      }
    }
    TR2(9);
  }
  if (!has2) {
    if (w == 0) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
    return;
  }

  // The slab of U: asked for only now, after this workgroup's share of stage 1 (and of the mix), because
  // a wave that queues this many loads is held up until most of them have been accepted, and the
  // work heading the dependency chain must not sit behind that.
  issue_prefetch(pf_lo, D2_PF);

  // ---- stage-2 activations: this slab's slice of z, polled from the tagged pairs into LDS ---------------
  __syncthreads();                                   // earlier uses of a_s and red are over
  TR2(3);
  {
    const int pairs = kcur2 >> 1;
    const int total = M * pairs;
    __amdgpu_buffer_rsrc_t zr = __builtin_amdgcn_make_buffer_rsrc(p.zt, 0, 0x7fffffff, 0x00020000);
    for (int base = 0; base < total; base += 256 * 4) {
      u32x4 v[4];
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = base + u * 256 + tid;
          if (idx < total) {
            const int m = idx / pairs, kp = idx - m * pairs;
            const uint32_t off = (uint32_t)((((int64_t)zi * M + m) * p.R + k0_2 + 2 * kp) * 8);
            v[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(zr, off, 0, 17));
            ok = ok && v[u][1] == epoch && v[u][3] == epoch;
          } else {
            v[u] = u32x4{0u, 0u, 0u, 0u};
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = base + u * 256 + tid;
        if (idx < total) {
          const int m = idx / pairs, kp = idx - m * pairs;
          a_s[m * KLD + 2 * kp] = __uint_as_float(v[u][0]);
          a_s[m * KLD + 2 * kp + 1] = __uint_as_float(v[u][2]);
        }
      }
    }
    // zero what the products below touch beyond the real data: rows m >= M and k in [kcur2, kpad2)
    const int kpad2 = p.kpad2;
    for (int idx = tid; idx < MT * kpad2; idx += 256) {
      const int m = idx / kpad2, k = idx - m * kpad2;
      if (m >= M || k >= kcur2) a_s[m * KLD + k] = 0.0f;
    }
  }
  __syncthreads();
  TR2(4);

  if (p.u_nk) {
    // ---- stage 2, U (bo, q, r): out[m, i Q + row] = sum_k z[m][k] U_i[row, k]; one wave per row, lanes along k ----
    if constexpr (WB == 16) {
      const int lane = tid & 63;
      const int KL = 1 << p.kl_log2;
      T* outp = reinterpret_cast<T*>(p.out);
      float racc[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) racc[m] = 0.0f;
#pragma unroll
      for (int u = 0; u < D2_PF; ++u) {
        if (u < p.pfn) {
          float wv[8];
          cvtw<T, 16>(pf[u], wv);
          const int c = u & (KL - 1);
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const f32x4 za = *reinterpret_cast<const f32x4*>(&a_s[m * KLD + c * 512 + lane * 8]);
            const f32x4 zb = *reinterpret_cast<const f32x4*>(&a_s[m * KLD + c * 512 + lane * 8 + 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e) racc[m] = fmaf(za[e], wv[e], racc[m]);
#pragma unroll
            for (int e = 0; e < 4; ++e) racc[m] = fmaf(zb[e], wv[4 + e], racc[m]);
          }
          if (c == KL - 1) {                               // the row is complete: add the 64 lanes, lane 0 stores
            const int row = nk_row0 + (u >> p.kl_log2);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const float tot = wave_sum(racc[m]);
              racc[m] = 0.0f;
              if (lane == 0 && row < p.Q && row < (nc2 + 1) * 4 * p.rpw && m < M)
                outp[(int64_t)m * p.ldo + (int64_t)i2 * p.o_bs + (int64_t)row * p.o_ns] = TypeTraits<T>::from_f32(tot);
            }
          }
        }
      }
    }
    TR2(7);
    if (w == 0) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
    return;
  }

  // ---- stage 2: out[m, i Q + n] = sum_k z[m][k] U_i[k, n] ---------------------------------------
  float acc[MT][EPL];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[m][e] = 0.0f;
  if constexpr (MT * EPL <= 32) {
    // The activations of all register-resident rows are read from LDS up front (one wait), so the products below
    // run back to back instead of paying an LDS round trip per row.  Slots at or beyond pfn are read but not used.
    float av[MT][D2_PF];
#pragma unroll
    for (int u = 0; u < D2_PF; ++u)
#pragma unroll
      for (int m = 0; m < MT; ++m) av[m][u] = a_s[m * KLD + ((rs2 + u * rpp2) & (KLD - 1))];   // zero beyond the slice
#pragma unroll
    for (int u = 0; u < D2_PF; ++u) {
      if (u < p.pfn) {
        float wv[EPL];
        cvtw<T, WB>(pf[u], wv);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(av[m][u], wv[e], acc[m][e]);
      }
    }
  } else {                                             // wide accumulators: no registers to spare for that
#pragma unroll
    for (int u = 0; u < D2_PF; ++u) {
      const int k = rs2 + u * rpp2;
      if (u < p.pfn) {
        float wv[EPL];
        cvtw<T, WB>(pf[u], wv);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float a = a_s[m * KLD + k];            // zero beyond the slice
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(a, wv[e], acc[m][e]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  {
    // rows the registers did not hold, in full batches (rows past the end meet a zero activation)
    const int rows_left = kcur2 - p.pfn * rpp2;
    const int nb = rows_left > 0 ? ((rows_left + rpp2 - 1) / rpp2 + D2_UNR - 1) / D2_UNR : 0;
    for (int bi = 0; bi < nb; ++bi) {
      u32x4 raw[D2_UNR];
#pragma unroll
      for (int u = 0; u < D2_UNR; ++u)
        raw[u] = ldw16(ubuf, uoff, (uint32_t)(p.pfn + bi * D2_UNR + u) * ustep);
#pragma unroll
      for (int u = 0; u < D2_UNR; ++u) {
        float wv[EPL];
        cvtw<T, WB>(raw[u], wv);
        const int k = rs2 + (p.pfn + bi * D2_UNR + u) * rpp2;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float a = a_s[m * KLD + k];
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[m][e] = fmaf(a, wv[e], acc[m][e]);
        }
      }
    }
  }
  TR2(5);
  float tot[MT][2];
  wg_reduce<MT, EPL>(acc, lpr2, cv2, red, NC2, tot);
  TR2(6);
  T* outp = reinterpret_cast<T*>(p.out);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int col = tid + h * 256;
    const int gn = n0_2 + col;
    if (col < NC2 && gn < p.Q) {
      if (ksi2 != 0) {                                // a producer of partial sums
#pragma unroll
        for (int m = 0; m < MT; ++m)
          if (m < M) st_tag(&p.opart[(((int64_t)(ksi2 - 1) * p.bo + i2) * M + m) * p.Q + gn], tot[m][h], epoch);
      } else {                                        // the slab of k-slice 0 adds the others in order
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          if (m < M) {
            float v = tot[m][h];
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
                __builtin_amdgcn_s_sleep(1);
              }
              v += __uint_as_float((unsigned)pv);
            }
            if (WB != 16) v *= (float)p.u_scales[(int64_t)i2 * p.Q + gn];                      // per-output scale of the codes of U
            outp[(int64_t)m * p.ldo + (int64_t)i2 * p.o_bs + (int64_t)gn * p.o_ns] = TypeTraits<T>::from_f32(v);
          }
        }
      }
    }
  }
  TR2(7);
  if (w == 0) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
}


// ---- matrix-core variant: up to 16 token rows --------------------------------------------------
// Same roles and hand-overs as decode2_kernel; the products run on v_mfma_f32_16x16x32.  Column
// chunks are 128 wide (16 lanes x 8), a lane loads 8 consecutive rows of its 8 columns per batch
// (a batch of a workgroup = 128 rows), transposes the 8x8 block in registers into eight B
// fragments, and the activations - staged in LDS as [16][k] of T - are the A fragment.  z crosses
// workgroups as {two T values, epoch} pairs (half the bytes of fp32 pairs: a slab's slice of z
// is 16 x 512 values at M = 16).
constexpr int DM_ROWS = 128;          // rows per batch of a workgroup
constexpr int DM_PF = 32;             // loads of the U slab kept in registers (4 batches)
constexpr int DM_KMAX = 1024;         // deepest staged slice
constexpr int DM_MC = 4;              // token rows per mix item

template <typename T>
__device__ __forceinline__ void dm_batch(const u32x4 (&cur)[8], const T* a_s, int ald, int cv, int rs, int kbase, f32x4 (&acc)[8]) {
  using V8 = typename TypeTraits<T>::vec8;
  const V8 af = *reinterpret_cast<const V8*>(&a_s[cv * ald + kbase + rs * 8]);     // row m = lane % 16, k = 8 (lane / 16) ..
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    u32x4 bb;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      bb[q] = __builtin_amdgcn_perm(cur[2 * q + 1][e >> 1], cur[2 * q][e >> 1], (e & 1) ? 0x07060302u : 0x05040100u);
    acc[e] = TypeTraits<T>::mfma16(af, __builtin_bit_cast(V8, bb), acc[e]);
  }
}

// The same batch when the weights are stored (n, k): load e is row n = column e of the lane's 8 at the lane's 8 consecutive k.
template <typename T>
__device__ __forceinline__ void dm_batch_nk(const u32x4 (&cur)[8], const T* a_s, int ald, int cv, int rs, int kbase, f32x4 (&acc)[8]) {
  using V8 = typename TypeTraits<T>::vec8;
  const V8 af = *reinterpret_cast<const V8*>(&a_s[cv * ald + kbase + rs * 8]);
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = TypeTraits<T>::mfma16(af, __builtin_bit_cast(V8, cur[e]), acc[e]);
}

// Two int8 codes sitting in bytes 0 and 2 of t (bytes 1 and 3 zero) -> two T values in one register.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <typename T>
__device__ __forceinline__ uint32_t cvt_pair_i8(uint32_t t) {
  if constexpr (sizeof(T) == 2 && __is_same(T, f16)) {
    // 0x6400 | (code ^ 0x80) is the half 1024 + (code + 128); one packed subtraction gives the code exactly
    const f16x2 v = __builtin_bit_cast(f16x2, t ^ 0x64806480u) - f16x2{(f16)1152.0f, (f16)1152.0f};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    return pack2<T>((float)(int8_t)(t & 0xffu), (float)(int8_t)((t >> 16) & 0xffu));
  }
}
// The batch for int8 codes stored (k, n): load u is row k + u of the lane's 8 columns, 8 bytes.  Fragment e takes byte e of
// rows 2q and 2q + 1 with one byte permute, which is the transpose and the widening to two-byte slots at once.
template <typename T>
__device__ __forceinline__ void dm_batch_i8(const u32x2 (&cur)[8], const T* a_s, int ald, int cv, int rs, int kbase, f32x4 (&acc)[8]) {
  using V8 = typename TypeTraits<T>::vec8;
  const V8 af = *reinterpret_cast<const V8*>(&a_s[cv * ald + kbase + rs * 8]);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t sel = 0x0c000c00u | ((4u + (e & 3)) << 16) | (uint32_t)(e & 3);
    u32x4 bb;
#pragma unroll
    for (int q = 0; q < 4; ++q) bb[q] = cvt_pair_i8<T>(__builtin_amdgcn_perm(cur[2 * q + 1][e >> 2], cur[2 * q][e >> 2], sel));
    acc[e] = TypeTraits<T>::mfma16(af, __builtin_bit_cast(V8, bb), acc[e]);
  }
}
// Two int4 codes (two's complement nibbles) sitting in bytes 0 and 2 of t -> two T values in one register.
template <typename T>
__device__ __forceinline__ uint32_t cvt_pair_i4(uint32_t t) {
  if constexpr (sizeof(T) == 2 && __is_same(T, f16)) {
    // 0x6400 | (nibble ^ 8) is the half 1024 + (code + 8)
    const f16x2 v = __builtin_bit_cast(f16x2, t ^ 0x64086408u) - f16x2{(f16)1032.0f, (f16)1032.0f};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    return pack2<T>((float)((int)((t & 0xfu) ^ 8u) - 8), (float)((int)(((t >> 16) & 0xfu) ^ 8u) - 8));
  }
}
// The batch for packed int4 codes stored (k, n), even column in the low nibble: load u is row k + u of the lane's 8 columns,
// 4 bytes.  Each row is split into its even and odd columns as bytes; from there it is the int8 scheme.
template <typename T>
__device__ __forceinline__ void dm_batch_i4(const uint32_t (&cur)[8], const T* a_s, int ald, int cv, int rs, int kbase, f32x4 (&acc)[8]) {
  using V8 = typename TypeTraits<T>::vec8;
  const V8 af = *reinterpret_cast<const V8*>(&a_s[cv * ald + kbase + rs * 8]);
  uint32_t ev[8], od[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) { ev[u] = cur[u] & 0x0f0f0f0fu; od[u] = (cur[u] >> 4) & 0x0f0f0f0fu; }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int c = e >> 1;
    const uint32_t sel = 0x0c000c00u | ((4u + c) << 16) | (uint32_t)c;
    u32x4 bb;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      bb[q] = cvt_pair_i4<T>((e & 1) ? __builtin_amdgcn_perm(od[2 * q + 1], od[2 * q], sel) : __builtin_amdgcn_perm(ev[2 * q + 1], ev[2 * q], sel));
    acc[e] = TypeTraits<T>::mfma16(af, __builtin_bit_cast(V8, bb), acc[e]);
  }
}
// one lane's piece of a weight row: 8 columns = 16 bytes of two-byte values, 8 bytes of int8 codes or 4 bytes of int4 codes
template <int WB> struct DmLoad { using type = u32x4; };
template <> struct DmLoad<8> { using type = u32x2; };
template <> struct DmLoad<4> { using type = uint32_t; };
template <int WB>
__device__ __forceinline__ typename DmLoad<WB>::type ldw8(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  if constexpr (WB == 8) return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 2));
  else if constexpr (WB == 4) return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 2);
  else return ldw16(r, voff, soff);
}

template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  typedef T T2 __attribute__((ext_vector_type(2)));
  T2 v = {TypeTraits<T>::from_f32(a), TypeTraits<T>::from_f32(b)};
  return __builtin_bit_cast(uint32_t, v);
}

template <typename T, int WB>
__global__ __launch_bounds__(256, 2) void decode2m_kernel(Decode2Params p) {
  static_assert(WB == 16 || WB == 8 || WB == 4, "two-byte weights, int8 codes or packed int4 codes");
  constexpr int PFN = WB == 16 ? DM_PF : 2 * DM_PF;    // loads of the U slab kept in registers (codes: a whole 1024-row slab)
  using LV = typename DmLoad<WB>::type;
  __shared__ __attribute__((aligned(16))) T a_s[16 * (DM_KMAX + 8)];
  __shared__ __attribute__((aligned(16))) float red[4 * 4 * 64 * 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cv = lane & 15, kg = lane >> 4, rs = wave * 4 + kg;
  const int w = blockIdx.x, G = gridDim.x;
  const int M = p.M;
  TR2(0);

  // (a plain, cached load: the word was last written before this kernel began, and hundreds of workgroups asking one
  // address for a device-scope copy would queue up at a single memory channel - with every later load of theirs behind it)
  unsigned epoch = *reinterpret_cast<const volatile unsigned*>(p.epoch_word) + 1u;
  if (epoch == 0u) epoch = 1u;
  auto check_in = [&]() {
    if (tid == 0) {
      asm volatile("" ::"v"(epoch) : "memory");
      (void)__hip_atomic_fetch_add(&p.arrive_word[(w % D2_SHARDS) * 64], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  // ---- stage-2 slab -------------------------------------------------------------------------------
  const int item2 = G - 1 - w;
  const bool has2 = item2 < p.items2;
  const int nc2 = has2 ? item2 % p.nch2 : 0;
  const int t2 = has2 ? item2 / p.nch2 : 0;
  const int i2 = t2 % p.bo, ksi2 = t2 / p.bo;
  const int zi = p.zrep > 1 ? nc2 % p.zrep : i2;     // which published copy of z this slab reads
  const int k0_2 = ksi2 * p.kc2;
  const int kcur2 = min(p.kc2, p.R - k0_2);
  const int n0_2 = nc2 * 128;
  const int n2 = n0_2 + cv * 8;
  const bool col_ok2 = n2 < p.Q;
  const __amdgpu_buffer_rsrc_t ubuf = wbuf(p.U, (uint32_t)((int64_t)p.bo * p.R * p.Q * WB / 8));
  // U (bo, r, q): load u of a batch is row k + u of the lane's 8 columns.  U (bo, q, r): load u is row q = column u of
  // the lane's 8, at the lane's 8 consecutive k - already a B fragment, so no transpose follows.
  const uint32_t uoff = p.u_nk ? (uint32_t)((((int64_t)i2 * p.Q + (col_ok2 ? n2 : 0)) * p.R + k0_2 + rs * 8) * 2)
                               : (uint32_t)((((int64_t)i2 * p.R + k0_2 + rs * 8) * p.Q + (col_ok2 ? n2 : 0)) * WB / 8);
  const uint32_t urow = (uint32_t)p.Q * (uint32_t)WB / 8u;
  auto u_soff = [&](int batch, int u) -> uint32_t {
    return p.u_nk ? (uint32_t)((u * p.R + batch * DM_ROWS) * 2) : (uint32_t)(batch * DM_ROWS + u) * urow;
  };
  LV pf[PFN];
  auto issue_prefetch = [&]() {
#pragma unroll
    for (int u = 0; u < PFN; ++u) {
      if (u < p.pfn) {
        if (u >= 4 && p.pf_depth == 4) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
        else if (u >= 8 && p.pf_depth == 8) asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
        else if (u >= 16 && p.pf_depth == 16) asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        pf[u] = ldw8<WB>(ubuf, uoff, u_soff(u >> 3, u & 7));
      }
    }
  };

  // Reduction of the four waves' fragments and hand-out of the totals: emit(h, e, l, v) receives,
  // for half h and fragment e, the four rows m = 4 (l / 16) + i of column 8 (l % 16) + 4 h + e.
  auto reduce_emit = [&](f32x4 (&acc)[8], auto&& emit) {
    f32x4 vh[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<f32x4*>(&red[((wave * 4 + e) * 64 + lane) * 4]) = acc[h * 4 + e];
      __syncthreads();
      const int e = tid >> 6, l = tid & 63;
      f32x4 v = *reinterpret_cast<const f32x4*>(&red[((0 * 4 + e) * 64 + l) * 4]);
      v += *reinterpret_cast<const f32x4*>(&red[((1 * 4 + e) * 64 + l) * 4]);
      v += *reinterpret_cast<const f32x4*>(&red[((2 * 4 + e) * 64 + l) * 4]);
      v += *reinterpret_cast<const f32x4*>(&red[((3 * 4 + e) * 64 + l) * 4]);
      vh[h] = v;
    }
    const int e = tid >> 6, l = tid & 63;
    emit((l & 15) * 8 + e, (l >> 4) * 4, vh);                       // columns col and col + 4
  };

  // ---- mix role: S of this thread's (i, r), asked for first -------------------------------------------
  const int nrc = (p.R + (1 << p.rch_log2) - 1) >> p.rch_log2;
  float sv[16];
  if (w < p.itemsM) {
    const int g = min(tid >> p.rch_log2, p.bo - 1);   // (replicas of a single output block all use S of block 0)
    const int r = min((w % nrc) * (1 << p.rch_log2) + (tid & ((1 << p.rch_log2) - 1)), p.R - 1);
    const T* Sp = reinterpret_cast<const T*>(p.S);
    if (Sp) {                                           // one uniform branch, then unconditional loads
#pragma unroll
      for (int u = 0; u < 16; ++u)
        sv[u] = TypeTraits<T>::to_f32(Sp[(int64_t)g * p.s_si + (int64_t)min(u, p.b - 1) * p.s_sj + (int64_t)r * p.s_sr]);
    } else {
#pragma unroll
      for (int u = 0; u < 16; ++u) sv[u] = 1.0f;
    }
  }

  // ---- stage 1 -----------------------------------------------------------------------------------
  if (w < p.items1) {
    const int nc1 = w % p.nch1;
    const int t1 = w / p.nch1;
    const int j = t1 % p.b, ks = t1 / p.b;
    const int k0 = ks * p.kc1, kc = min(p.kc1, p.P - k0);
    const int n0 = nc1 * 128, n = n0 + cv * 8;
    const bool col_ok = n < p.R;
    const __amdgpu_buffer_rsrc_t vbuf = wbuf(p.V, (uint32_t)((int64_t)p.b * p.P * p.R * WB / 8));
    const uint32_t voff = (uint32_t)((((int64_t)j * p.P + k0 + rs * 8) * p.R + (col_ok ? n : 0)) * WB / 8);
    const uint32_t vrow = (uint32_t)p.R * (uint32_t)WB / 8u;
    const int nbatch = (kc + DM_ROWS - 1) / DM_ROWS;
    const int kpad = nbatch * DM_ROWS, ald = kpad + 8;
    LV raw[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) raw[u] = ldw8<WB>(vbuf, voff, (uint32_t)u * vrow);
    // activations straight into LDS as T (zero outside the slice and beyond M)
    const T* xp = reinterpret_cast<const T*>(p.x);
    if (p.x_vec) {                                               // 16-byte pieces: one or two per thread
      const int pieces = kpad >> 3;
      for (int idx = tid; idx < 16 * pieces; idx += 256) {
        const int m = idx / pieces, ka = (idx - m * pieces) * 8;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (m < M && ka < kc) v = *reinterpret_cast<const u32x4*>(&xp[(int64_t)m * p.ldx + (int64_t)j * p.P + k0 + ka]);
        if (m < M && ka + 8 > kc && ka < kc) {                   // piece straddling the end of the slice
          uint16_t* h = reinterpret_cast<uint16_t*>(&v);
#pragma unroll
          for (int e = 0; e < 8; ++e) if (ka + e >= kc) h[e] = 0;
        }
        *reinterpret_cast<u32x4*>(&a_s[m * ald + ka]) = v;
      }
    } else {
      for (int idx = tid; idx < 16 * kpad; idx += 256) {
        const int m = idx / kpad, ka = idx - m * kpad;
        T v = TypeTraits<T>::from_f32(0.0f);
        if (m < M && ka < kc) v = xp[(int64_t)m * p.ldx + (int64_t)j * p.P + k0 + ka];
        a_s[m * ald + ka] = v;
      }
    }
    check_in();
    __syncthreads();
    f32x4 acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int bi = 0; bi < nbatch; ++bi) {
      LV cur[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) cur[u] = raw[u];
      if (bi + 1 < nbatch) {
#pragma unroll
        for (int u = 0; u < 8; ++u) raw[u] = ldw8<WB>(vbuf, voff, (uint32_t)((bi + 1) * DM_ROWS + u) * vrow);
      }
      if constexpr (WB == 8) dm_batch_i8<T>(cur, a_s, ald, cv, rs, bi * DM_ROWS, acc);
      else if constexpr (WB == 4) dm_batch_i4<T>(cur, a_s, ald, cv, rs, bi * DM_ROWS, acc);
      else dm_batch<T>(cur, a_s, ald, cv, rs, bi * DM_ROWS, acc);
    }
    TR2(1);
    // y crosses workgroups as {two T values (ranks 2c, 2c + 1), epoch} pairs.  The totals go through LDS once more so
    // that a wave stores 64 consecutive pairs of one token row (512 contiguous bytes) instead of 8-byte pieces 64 bytes apart.
    constexpr int YLD = 130;
    reduce_emit(acc, [&](int col, int m0, const f32x4 (&vh)[2]) {
      __syncthreads();                                            // every thread has read its sums out of red
      float vsc[2] = {1.0f, 1.0f};                                // int8 codes of V: one scale per rank
      if constexpr (WB != 16) {
#pragma unroll
        for (int h = 0; h < 2; ++h) vsc[h] = (float)p.v_scales[(int64_t)j * p.R + min(n0 + col + 4 * h, p.R - 1)];
      }
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[(m0 + i) * YLD + col + 4 * h] = vh[h][i] * vsc[h];
    });
    __syncthreads();
    {
      const int cp = tid & 63, mq = (tid >> 6) * 4;
      const int gn = n0 + 2 * cp;
      if (gn < p.R) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int m = mq + i;
          if (m < M) {
            const unsigned long long v = ((unsigned long long)epoch << 32) |
                                         pack2<T>(red[m * YLD + 2 * cp], (gn + 1 < p.R) ? red[m * YLD + 2 * cp + 1] : 0.0f);
            __hip_atomic_store(&p.ypart[(((int64_t)ks * p.b + j) * M + m) * (p.R >> 1) + (gn >> 1)], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
    }
    TR2(2);
  } else {
    check_in();
  }

  // ---- mix role: item = (chunk of RCH ranks, DM_MC token rows); z goes out as tagged pairs of T -----------
  if (w < p.itemsM) {
    __syncthreads();
    TR2(8);
    float* ys = reinterpret_cast<float*>(a_s);                  // [DM_MC][256]
    const int RCH = 1 << p.rch_log2;
    const int g = tid >> p.rch_log2, rr = tid & (RCH - 1);
    const int r = (w % nrc) * RCH + rr;
    const int mbase = (w / nrc) * DM_MC;
    const bool perm = p.perm_per > 0;                  // Monarch: z[l][r] = y[r / per][l * per + r % per]
    const int yj = perm ? r / p.perm_per : g;
    const int yr = perm ? g * p.perm_per + r % p.perm_per : r;
    const bool live = (perm ? g < p.bo : g < p.b) && r < p.R;          // fetches y of input block yj
    const bool live_o = g < (p.zrep > 1 ? p.zrep : p.bo) && r < p.R;   // emits z of output block (or replica) g
    const T* Sp = reinterpret_cast<const T*>(p.S);
    float ysum[DM_MC];
#pragma unroll
    for (int m = 0; m < DM_MC; ++m) ysum[m] = 0.0f;
    if (live) {
      unsigned long long yv[4][DM_MC];
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
          for (int m = 0; m < DM_MC; ++m) {
            if (ks < p.ks1 && mbase + m < M) {
              yv[ks][m] = ld_tag(&p.ypart[(((int64_t)ks * p.b + yj) * M + mbase + m) * (p.R >> 1) + (yr >> 1)]);
              ok = ok && ((unsigned)(yv[ks][m] >> 32) == epoch);
            } else {
              yv[ks][m] = 0ull;
            }
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int m = 0; m < DM_MC; ++m) {                          // this thread's rank is one half of the pair
          typedef T T2 __attribute__((ext_vector_type(2)));
          const T2 pr = __builtin_bit_cast(T2, (unsigned)yv[ks][m]);
          ysum[m] += TypeTraits<T>::to_f32((yr & 1) ? pr[1] : pr[0]);
        }
    }
#pragma unroll
    for (int m = 0; m < DM_MC; ++m) ys[m * 256 + tid] = ysum[m];
    __syncthreads();
#pragma unroll
    for (int m = 0; m < DM_MC; ++m) {
      float z = perm ? ysum[m] : 0.0f;
      if (live_o && !perm) {
#pragma unroll
        for (int u = 0; u < 16; ++u) z = fmaf((u < p.b) ? sv[u] : 0.0f, ys[m * 256 + min(u, p.b - 1) * RCH + rr], z);
        for (int jx = 16; jx < p.b; ++jx)
          z = fmaf(Sp ? TypeTraits<T>::to_f32(Sp[(int64_t)min(g, p.bo - 1) * p.s_si + (int64_t)jx * p.s_sj + (int64_t)r * p.s_sr]) : 1.0f, ys[m * 256 + jx * RCH + rr], z);
      }
      const float zn = __shfl_down(z, 1, 64);                    // rank r + 1 (same i: RCH is even)
      if (live_o && (rr & 1) == 0 && mbase + m < M) {
        const unsigned long long v = ((unsigned long long)epoch << 32) | pack2<T>(z, (r + 1 < p.R) ? zn : 0.0f);
        __hip_atomic_store(&p.zt[((int64_t)g * M + mbase + m) * (p.R >> 1) + (r >> 1)], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    TR2(9);
  }
  if (!has2) {
    if (w == 0) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
    return;
  }

  issue_prefetch();

  // ---- stage-2 activations: z slice -> LDS as T ----------------------------------------------------------
  __syncthreads();
  TR2(3);
  const int kpad2 = p.kpad2, ald2 = kpad2 + 8;
  {
    const int quads = kcur2 >> 2;                                 // 16-byte units (4 ranks) per token row
    const int total = M * quads;
    __amdgpu_buffer_rsrc_t zr = __builtin_amdgcn_make_buffer_rsrc(p.zt, 0, 0x7fffffff, 0x00020000);
    for (int base = 0; base < total; base += 256 * 8) {
      u32x4 v[8];
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int idx = base + u * 256 + tid;
          if (idx < total) {
            const int m = idx / quads, kq = idx - m * quads;
            const uint32_t off = (uint32_t)((((int64_t)zi * M + m) * (p.R >> 1) + ((k0_2 + 4 * kq) >> 1)) * 8);
            v[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(zr, off, 0, 17));
            ok = ok && v[u][1] == epoch && v[u][3] == epoch;
          } else {
            v[u] = u32x4{0u, 0u, 0u, 0u};
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = base + u * 256 + tid;
        if (idx < total) {
          const int m = idx / quads, kq = idx - m * quads;
          uint32_t* dst = reinterpret_cast<uint32_t*>(&a_s[m * ald2 + 4 * kq]);
          dst[0] = v[u][0];
          dst[1] = v[u][2];
        }
      }
    }
    for (int idx = tid; idx < 16 * kpad2; idx += 256) {           // zero rows beyond M and ranks beyond the slice
      const int m = idx / kpad2, k = idx - m * kpad2;
      if (m >= M || k >= kcur2) a_s[m * ald2 + k] = TypeTraits<T>::from_f32(0.0f);
    }
  }
  __syncthreads();
  TR2(4);

  // ---- stage 2 --------------------------------------------------------------------------------------
  f32x4 acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int bq = 0; bq < PFN / 8; ++bq) {
    if (bq * 8 < p.pfn) {
      LV cur[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) cur[u] = pf[bq * 8 + u];
      if constexpr (WB == 8) dm_batch_i8<T>(cur, a_s, ald2, cv, rs, bq * DM_ROWS, acc);
      else if constexpr (WB == 4) dm_batch_i4<T>(cur, a_s, ald2, cv, rs, bq * DM_ROWS, acc);
      else if (p.u_nk) dm_batch_nk<T>(cur, a_s, ald2, cv, rs, bq * DM_ROWS, acc);
      else dm_batch<T>(cur, a_s, ald2, cv, rs, bq * DM_ROWS, acc);
    }
  }
  {
    // Deeper slabs: the rest is asked for in one go (up to DM_PF more loads per lane, into the registers the
    // products above have freed), so it costs one trip to memory and not one per batch.  The loads are
    // unconditional: a batch past the end of the slab gets an offset beyond the buffer, which reads as zero
    // without touching memory, and is not multiplied.
    const int nbq = (kcur2 + DM_ROWS - 1) / DM_ROWS;
    for (int b0 = p.pfn / 8; b0 < nbq; b0 += PFN / 8) {
#pragma unroll
      for (int bq = 0; bq < PFN / 8; ++bq) {
        const bool in_slab = b0 + bq < nbq;
        const uint32_t vo = in_slab ? uoff : 0x80000000u;           // the per-lane offset is what the bounds check sees
#pragma unroll
        for (int u = 0; u < 8; ++u) pf[bq * 8 + u] = ldw8<WB>(ubuf, vo, in_slab ? u_soff(b0 + bq, u) : 0u);
      }
#pragma unroll
      for (int bq = 0; bq < PFN / 8; ++bq) {
        if (b0 + bq < nbq) {
          LV cur[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) cur[u] = pf[bq * 8 + u];
          if constexpr (WB == 8) dm_batch_i8<T>(cur, a_s, ald2, cv, rs, (b0 + bq) * DM_ROWS, acc);
          else if constexpr (WB == 4) dm_batch_i4<T>(cur, a_s, ald2, cv, rs, (b0 + bq) * DM_ROWS, acc);
          else if (p.u_nk) dm_batch_nk<T>(cur, a_s, ald2, cv, rs, (b0 + bq) * DM_ROWS, acc);
          else dm_batch<T>(cur, a_s, ald2, cv, rs, (b0 + bq) * DM_ROWS, acc);
        }
      }
    }
  }
  TR2(5);
  T* outp = reinterpret_cast<T*>(p.out);
  reduce_emit(acc, [&](int col, int m0, const f32x4 (&vh)[2]) {
    if (ksi2 != 0) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int gn = n0_2 + col + 4 * h;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (gn < p.Q && m0 + i < M) st_tag(&p.opart[(((int64_t)(ksi2 - 1) * p.bo + i2) * M + m0 + i) * p.Q + gn], vh[h][i], epoch);
      }
      return;
    }
    float tot[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) tot[h][i] = vh[h][i];
    if (p.ks2 > 1) {                                                // all partial sums of this thread's 8 outputs in one go
      unsigned long long pv[3][2][4];
      unsigned spins = 0;
      while (true) {
        bool ok = true;
#pragma unroll
        for (int ks = 1; ks < 4; ++ks) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int gn = n0_2 + col + 4 * h;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (ks < p.ks2 && gn < p.Q && m0 + i < M) {
                pv[ks - 1][h][i] = ld_tag(&p.opart[(((int64_t)(ks - 1) * p.bo + i2) * M + m0 + i) * p.Q + gn]);
                ok = ok && ((unsigned)(pv[ks - 1][h][i] >> 32) == epoch);
              } else {
                pv[ks - 1][h][i] = 0ull;
              }
            }
          }
        }
        if (ok) break;
        if (++spins > p.spin_limit) {
          __hip_atomic_store(p.err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int ks = 0; ks < 3; ++ks)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) tot[h][i] += __uint_as_float((unsigned)pv[ks][h][i]);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int gn = n0_2 + col + 4 * h;
      float usc = 1.0f;                                              // int8 codes of U: one scale per output column
      if constexpr (WB != 16) usc = (float)p.u_scales[(int64_t)i2 * p.Q + min(gn, p.Q - 1)];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (gn < p.Q && m0 + i < M) outp[(int64_t)(m0 + i) * p.ldo + (int64_t)i2 * p.o_bs + (int64_t)gn * p.o_ns] = TypeTraits<T>::from_f32(tot[h][i] * usc);
    }
  });
  TR2(7);
  if (w == 0) finish_epoch(p.arrive_word, p.epoch_word, p.err_word, epoch, G, p.spin_limit);
}

// ---- dense layer at up to 16 token rows ---------------------------------------------------------------
// out = x W with W (K, N) row-major: nothing crosses workgroups before the products, so this is the slab stage of the
// kernel above on its own.  A workgroup owns 128 columns and a slice of up to 1024 rows of W: the slice of x goes to LDS,
// the slab streams through four batches of registers (32 loads per lane in flight, a consumed batch is refilled at
// once), the products run on the matrix cores.  With one slice the result is stored as T; otherwise every slice
// writes fp32 partial sums P[slice][m][n] with plain stores and dense_slab_reduce_kernel adds them in fixed order
// in a second launch: no spinning, no limit on the grid.
struct DenseSlabParams {
  const void* x; int64_t ldx; const void* W; void* out; int64_t ldo; float* part;
  int64_t sx, sw, so, ldw;                 // batches: element strides of x, W and out; row stride of W
  int M, K, N, nch, ks, kc, x_vec, batch;
};

template <typename T>
__global__ __launch_bounds__(256, 2) void dense_slab_kernel(DenseSlabParams p) {
  __shared__ __attribute__((aligned(16))) T a_s[16 * (DM_KMAX + 8)];
  __shared__ __attribute__((aligned(16))) float red[4 * 4 * 64 * 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cv = lane & 15, kg = lane >> 4, rs = wave * 4 + kg;
  const int nc = blockIdx.x % p.nch, tb = blockIdx.x / p.nch;
  const int bt = tb % p.batch, sl = tb / p.batch;
  const int k0 = sl * p.kc, kc = min(p.kc, p.K - k0);
  const int n0 = nc * 128, n = n0 + cv * 8;
  const bool col_ok = n < p.N;
  const int M = p.M;
  const __amdgpu_buffer_rsrc_t wb = wbuf(reinterpret_cast<const T*>(p.W) + (int64_t)bt * p.sw, (uint32_t)((int64_t)p.K * p.ldw * 2));
  const uint32_t woff = (uint32_t)((((int64_t)k0 + rs * 8) * p.ldw + (col_ok ? n : 0)) * 2);
  const uint32_t wrow = (uint32_t)p.ldw * 2u;
  const int nb = (kc + DM_ROWS - 1) / DM_ROWS;          // batches of 128 rows; rows past the end of W read as zero
  const int kpad = nb * DM_ROWS, ald = kpad + 8;
  u32x4 pf[DM_PF];
#pragma unroll
  for (int bq = 0; bq < DM_PF / 8; ++bq) {
    const uint32_t vo = bq < nb ? woff : 0x80000000u;   // a batch past the slice: offset beyond the buffer, reads as zero
#pragma unroll
    for (int u = 0; u < 8; ++u) pf[bq * 8 + u] = ldw16(wb, vo, bq < nb ? (uint32_t)(bq * DM_ROWS + u) * wrow : 0u);
  }
  // the slice of x as T, zero beyond M rows and beyond the slice
  const T* xp = reinterpret_cast<const T*>(p.x) + (int64_t)bt * p.sx;
  if (p.x_vec) {                                         // 16-byte pieces: every piece aligned and inside the row
    const int pieces = kpad >> 3;
    for (int idx = tid; idx < 16 * pieces; idx += 256) {
      const int m = idx / pieces, ka = (idx - m * pieces) * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (m < M && ka < kc) v = *reinterpret_cast<const u32x4*>(&xp[(int64_t)m * p.ldx + k0 + ka]);
      *reinterpret_cast<u32x4*>(&a_s[m * ald + ka]) = v;
    }
  } else {
    for (int idx = tid; idx < 16 * kpad; idx += 256) {
      const int m = idx / kpad, ka = idx - m * kpad;
      T v = TypeTraits<T>::from_f32(0.0f);
      if (m < M && ka < kc) v = xp[(int64_t)m * p.ldx + k0 + ka];
      a_s[m * ald + ka] = v;
    }
  }
  __syncthreads();
  f32x4 acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  // Straight-line code: the loads are unconditional (past the slice they cost nothing), only the products are skipped,
  // so the compiler can count the loads in flight instead of waiting for all of them at every branch.
#pragma unroll
  for (int bt = 0; bt < DM_KMAX / DM_ROWS; ++bt) {
    constexpr int NSLOT = DM_PF / 8;
    const int bq = bt % NSLOT;
    u32x4 cur[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) cur[u] = pf[bq * 8 + u];
    if (bt + NSLOT < DM_KMAX / DM_ROWS) {                  // refill the registers just read with the batch four ahead
      const int nxt = bt + NSLOT;
      const uint32_t vo = nxt < nb ? woff : 0x80000000u;
#pragma unroll
      for (int u = 0; u < 8; ++u) pf[bq * 8 + u] = ldw16(wb, vo, nxt < nb ? (uint32_t)(nxt * DM_ROWS + u) * wrow : 0u);
    }
    if (bt < nb) dm_batch<T>(cur, a_s, ald, cv, rs, bt * DM_ROWS, acc);
  }
  // sum of the four waves (they hold different rows of the slice), then thread (e, l) owns rows 4 (l / 16) .. + 3 of
  // columns 8 (l % 16) + e and + 4 of that
  f32x4 vh[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 4; ++e) *reinterpret_cast<f32x4*>(&red[((wave * 4 + e) * 64 + lane) * 4]) = acc[h * 4 + e];
    __syncthreads();
    const int e = tid >> 6, l = tid & 63;
    f32x4 v = *reinterpret_cast<const f32x4*>(&red[((0 * 4 + e) * 64 + l) * 4]);
    v += *reinterpret_cast<const f32x4*>(&red[((1 * 4 + e) * 64 + l) * 4]);
    v += *reinterpret_cast<const f32x4*>(&red[((2 * 4 + e) * 64 + l) * 4]);
    v += *reinterpret_cast<const f32x4*>(&red[((3 * 4 + e) * 64 + l) * 4]);
    vh[h] = v;
  }
  // through LDS once more so that a wave writes whole rows of the 128-column chunk
  constexpr int OLD = 132;
  __syncthreads();
  {
    const int e = tid >> 6, l = tid & 63, col = (l & 15) * 8 + e, m0 = (l >> 4) * 4;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(m0 + i) * OLD + col + 4 * h] = vh[h][i];
  }
  __syncthreads();
  {
    const int c4 = (tid & 31) * 4, mr = tid >> 5;        // 4 columns of rows mr and mr + 8
    const int gn = n0 + c4;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int m = mr + 8 * hh;
      if (m < M && gn < p.N) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(&red[m * OLD + c4]);
        if (p.ks > 1) {
          float* dst = &p.part[(((int64_t)sl * p.batch + bt) * M + m) * p.N + gn];
          if (gn + 3 < p.N && (p.N & 3) == 0) *reinterpret_cast<f32x4*>(dst) = v;
          else { for (int e = 0; e < 4; ++e) if (gn + e < p.N) dst[e] = v[e]; }
        } else {
          T* dst = &reinterpret_cast<T*>(p.out)[(int64_t)bt * p.so + (int64_t)m * p.ldo + gn];
          for (int e = 0; e < 4; ++e) if (gn + e < p.N) dst[e] = TypeTraits<T>::from_f32(v[e]);
        }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void dense_slab_reduce_kernel(const float* __restrict__ P, T* __restrict__ out, int64_t ldo, int64_t so,
                                                                 int M, int N, int ks, int batch) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)batch * M * N) return;
  const int n = (int)(idx % N);
  const int64_t t = idx / N;
  const int m = (int)(t % M), bt = (int)(t / M);
  // four slices are asked for together (one trip to memory, not one per slice) and added in slice order
  const int64_t sstride = (int64_t)batch * M * N;
  const float* src = P + ((int64_t)bt * M + m) * N + n;
  float v = 0.0f;
  int s = 0;
  for (; s + 4 <= ks; s += 4) {
    const float a0 = src[(int64_t)s * sstride], a1 = src[(int64_t)(s + 1) * sstride];
    const float a2 = src[(int64_t)(s + 2) * sstride], a3 = src[(int64_t)(s + 3) * sstride];
    v += a0; v += a1; v += a2; v += a3;
  }
  for (; s < ks; ++s) v += src[(int64_t)s * sstride];
  out[(int64_t)bt * so + (int64_t)m * ldo + n] = TypeTraits<T>::from_f32(v);
}

// ---- host side -----------------------------------------------------------------------------------
namespace {

template <typename T, int WB>
void* d2_kernel_mt(int MT) {
  switch (MT) {
    case 1: return (void*)decode2_kernel<T, 1, WB>;
    case 2: return (void*)decode2_kernel<T, 2, WB>;
    default: return (void*)decode2_kernel<T, 4, WB>;
  }
}
template <typename T>
void* d2_kernel(int MT, int wbits) {
  if (wbits == 8) return d2_kernel_mt<T, 8>(MT);
  if (wbits == 4) return d2_kernel_mt<T, 4>(MT);
  return d2_kernel_mt<T, 16>(MT);
}

}  // namespace

size_t decode2_region_bytes() { return (size_t)16 << 20; }
size_t decode2_plain_bytes() { return (size_t)8 << 20; }

bool decode2_applicable(const StreamBlastArgs& a) {
  const int enabled = option_value(OPT_DECODE2, 1);
  if (!enabled || a.split) return false;
  if (a.u_layout != BLR_U_RQ && !(a.u_layout == BLR_U_QR && a.wbits == 16)) return false;
  if (a.wbits != 16 && (a.wbits != 8 && a.wbits != 4)) return false;
  if (a.wbits != 16 && (!a.u_scales || !a.v_scales)) return false;
  if (a.dtype != BLR_F16 && a.dtype != BLR_BF16) return false;
  if (a.M < 1 || a.M > 16) return false;
  const int P = a.in_f / a.b, Q = a.out_f / (a.bo > 0 ? a.bo : a.b);
  if (a.r % 8 || Q % 8 || P < 1) return false;
  if (!aligned(a.U, 16) || !aligned(a.V, 16)) return false;
  if ((int64_t)a.r * a.out_f * 2 >= (1ll << 31) || (int64_t)a.r * a.in_f * 2 >= (1ll << 31)) return false;   // 32-bit buffer offsets
  return true;
}

int decode2m_blast_launch(const StreamBlastArgs& a, void* region, unsigned* epoch_word, unsigned* arrive_word,
                          unsigned* err_word, hipStream_t st);

// region: the fixed-place 16 MiB block of the workspace reserved for tagged pairs; ctrl3: three
// words on separate cache lines (epoch, arrivals, error).
int decode2_blast_launch(const StreamBlastArgs& a, void* region, void* plain, unsigned* epoch_word, unsigned* arrive_word,
                         unsigned* err_word, hipStream_t st) {
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int P = a.in_f / a.b, Q = a.out_f / bo, R = a.r, b = a.b, M = a.M;
  constexpr int rows_min_m = 2;
  if (M >= rows_min_m || a.wbits == 4 || a.rows_only) {   // (4-bit codes at one row too: 15.8 against 16.9 - 20.6 us on the single-row kernels)
    const int rc = decode_rows_launch(a, plain, decode2_plain_bytes(), st);
    if (rc != 1) return rc;
  }
  if (a.rows_only) { set_error("blast_q: code rows that are not whole 16-byte pieces need in_f / b, r and out_f / b to be multiples of 8 and at most 4096"); return BLR_ERR_UNSUPPORTED; }
  if (a.perm_per > 0) {
    // Monarch (few, wide blocks): the single-launch kernel where its stage 1 fits one batch of loads per item (11.3 against
    // about 12 us at 4096 -> 4096), the two launches for deeper input blocks (11008 -> 4096: input blocks of 2752 rows)
    int rc = decode3_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    if (rc != 1) return rc;
    rc = decode_pair_launch(a, plain, decode2_plain_bytes(), st);
    if (rc != 1) return rc;
  } else {
    int rc = decode_pair_launch(a, plain, decode2_plain_bytes(), st);
    if (rc != 1) return rc;
    rc = decode3_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    if (rc != 1) return rc;
  }
  constexpr int mfma_min_m = 5;
  if (M >= mfma_min_m && a.wbits == 16) return decode2m_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
  constexpr int q_mfma_min_m = 3;
  if ((M > 4 || M >= q_mfma_min_m) && a.wbits != 16) {   // below that, codes stay with the vector variant
    const int rc = decode2m_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    if (rc != 1 || M > 4) return rc;                     // a shape it declines at 3 or 4 rows is still the vector variant's
  }
  if (M > 4) return d2_bail(__LINE__);
  const int MT = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
  const int WBITS = a.wbits, EPL = 128 / WBITS;  // weights per 16-byte load
  const int kc_cap = D2_AS / MT - 256;           // the kernels pad a slice up to 255 rows with zeros
  void* fn = a.dtype == BLR_F16 ? d2_kernel<f16>(MT, WBITS) : d2_kernel<bf16>(MT, WBITS);

  static std::mutex mu;
  static std::map<void*, int> occ_cache;
  int occ = 0;
  {
    std::lock_guard<std::mutex> lk(mu);
    auto it = occ_cache.find(fn);
    if (it != occ_cache.end()) occ = it->second;
    else {
      hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, 256, 0);
      if (e != hipSuccess || occ < 1) { (void)hipGetLastError(); set_error("decode2: occupancy query failed"); return BLR_ERR_LAUNCH; }
      occ_cache[fn] = occ;
    }
  }
  const int cus = device_cus() > 0 ? device_cus() : 256;
  const int resident = (occ < 2 ? occ : 2) * cus;

  Decode2Params p = {};
  p.x = a.x; p.ldx = a.ldx; p.V = a.V; p.U = a.U; p.S = a.S; p.out = a.out; p.ldo = a.ldo;
  p.u_scales = (const f16*)a.u_scales; p.v_scales = (const f16*)a.v_scales;
  p.M = M; p.b = b; p.bo = bo; p.P = P; p.R = R; p.Q = Q;
  p.perm_per = a.perm_per; p.o_bs = a.out_ns ? a.out_bs : Q; p.o_ns = a.out_ns ? a.out_ns : 1;
  if (a.s_layout == BLR_S_JIR) { p.s_sj = (int64_t)b * R; p.s_si = R; p.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { p.s_sr = (int64_t)b * b; p.s_si = b; p.s_sj = 1; }
  else { p.s_si = (int64_t)b * R; p.s_sj = R; p.s_sr = 1; }
  const int lpr_cap = D2_NC_MAX / EPL;           // widest column chunk the reduction buffer holds

  if (a.u_layout == BLR_U_QR) {
    // stage 2 on U (bo, q, r): a wave takes rpw rows, a lane 8 of every 512 k; everything a lane loads stays in registers
    // shapes this geometry does not hold (rows of a wave times k pieces beyond the registers of a lane) go to the
    // matrix-core variant, which takes this layout at any M
    const int KL = (R + 511) / 512;
    if (KL != 1 && KL != 2 && KL != 4 && KL != 8) return decode2m_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    if (KL * 512 * MT > D2_AS) return decode2m_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    const int pf_cap = d2_pf(MT, 16);
    int rpw = (int)cdiv((int64_t)bo * Q, (int64_t)resident * 4);
    if (rpw < 1) rpw = 1;
    while ((int64_t)bo * cdiv(Q, 4 * rpw) > resident) ++rpw;
    if (rpw * KL > pf_cap) return decode2m_blast_launch(a, region, epoch_word, arrive_word, err_word, st);
    p.u_nk = 1; p.rpw = rpw; p.kl_log2 = ilog2(KL);
    p.lpr2_log2 = 4; p.nch2 = (int)cdiv(Q, 4 * rpw); p.ks2 = 1; p.kc2 = R; p.items2 = bo * p.nch2;
    p.pfn = rpw * KL; p.kpad2 = KL * 512;
  } else
  // stage 2: column chunks of 8 * lpr2 outputs; k split so that the slabs cover the resident grid
  {
    constexpr int ks_cap = 4;
    int lpr = 16 < lpr_cap ? 16 : lpr_cap;
    const int vecs = (Q + EPL - 1) / EPL;
    while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
    if (lpr > 64) lpr = 64;
    if (lpr < 4) lpr = 4;
    const int rpp = 256 / lpr;
    const int nch = (vecs + lpr - 1) / lpr;
    const int base = bo * nch;
    if (base > resident) return d2_bail(__LINE__);
    int ks = resident / base;
    if (ks > ks_cap) ks = ks_cap;
    if (ks > resident / base) ks = resident / base;
    if (ks < 1) ks = 1;
    int kc = (R + ks - 1) / ks;
    kc = (kc + rpp - 1) / rpp * rpp;
    if (kc > kc_cap) kc = kc_cap / rpp * rpp;
    if (kc < 1) return d2_bail(__LINE__);
    ks = (R + kc - 1) / kc;
    if (base * ks > resident) return d2_bail(__LINE__);
    int pfn = (kc + rpp - 1) / rpp;
    if (pfn > d2_pf(MT, WBITS)) pfn = d2_pf(MT, WBITS);
    const int left = (kc + rpp - 1) / rpp - pfn;     // loads per lane beyond the register-resident ones
    const int kpad2 = (pfn + (left > 0 ? (left + D2_UNR - 1) / D2_UNR * D2_UNR : 0)) * rpp;
    if (kpad2 > D2_AS / MT) return d2_bail(__LINE__);
    p.lpr2_log2 = ilog2(lpr); p.nch2 = nch; p.ks2 = ks; p.kc2 = kc; p.items2 = base * ks; p.pfn = pfn; p.kpad2 = kpad2;
  }
  // stage 1: column chunks of EPL * lpr1 ranks; k split only as far as needed to engage the chip
  {
    int lpr = 16 < lpr_cap ? 16 : lpr_cap;
    const int vecs = (R + EPL - 1) / EPL;
    while (lpr > 4 && lpr / 2 >= vecs) lpr /= 2;
    if (lpr > 64) lpr = 64;
    if (lpr > lpr_cap) lpr = lpr_cap;
    if (lpr < 4) lpr = 4;
    const int rpp = 256 / lpr;
    const int nch = (vecs + lpr - 1) / lpr;
    const int base = b * nch;
    if (base > resident) return d2_bail(__LINE__);
    // split k just far enough that a lane's share of a slice is one batch of loads
    const int ks_max = d2_ks1_max(MT);
    int ks = ((P + rpp - 1) / rpp + d2_unr1(MT) - 1) / d2_unr1(MT);
    if (ks > resident / base) ks = resident / base;
    // A workgroup that owns both a stage-1 item and a slab of U starts streaming its slab only after its stage-1
    // work and ends last: when a slightly coarser k split lets every item have a workgroup of its own, take it
    // (as long as a lane's share of a slice still fits two batches of loads).
    if (base + p.items2 <= resident && base * ks + p.items2 > resident) {
      const int ks_solo = (resident - p.items2) / base;
      if (((P + ks_solo - 1) / ks_solo + rpp - 1) / rpp <= 2 * d2_unr1(MT)) ks = ks_solo;
    }
    if (ks > ks_max) ks = ks_max;
    if (ks > (P + rpp - 1) / rpp) ks = (P + rpp - 1) / rpp;     // at least one load per lane
    if (ks < 1) ks = 1;
    int kc = (P + ks - 1) / ks;
    kc = (kc + rpp - 1) / rpp * rpp;
    if (kc > kc_cap) kc = kc_cap / rpp * rpp;
    if (kc < 1) return d2_bail(__LINE__);
    ks = (P + kc - 1) / kc;
    if (ks > ks_max || base * ks > resident) return d2_bail(__LINE__);
    const int unr1 = d2_unr1(MT);
    if (((kc + rpp - 1) / rpp + unr1 - 1) / unr1 * unr1 * rpp > D2_AS / MT) return d2_bail(__LINE__);   // zero padding must fit too
    p.lpr1_log2 = ilog2(lpr); p.nch1 = nch; p.ks1 = ks; p.kc1 = kc; p.items1 = base * ks;
  }
  {
    p.zrep = bo == 1 ? 16 : 1;
    int bp2 = 1;
    while (bp2 < b || bp2 < bo || bp2 < p.zrep) bp2 <<= 1;
    if (bp2 > 256) return d2_bail(__LINE__);
    const int rch = 256 / bp2;
    p.rch_log2 = ilog2(rch);
    p.itemsM = (R + rch - 1) / rch;
    if (p.itemsM > resident) return d2_bail(__LINE__);
    p.pf_depth = 4;
    p.pf_first = 0;
  }
  const size_t ybytes = align_up((size_t)p.ks1 * b * M * R * 8, 256), zbytes = align_up((size_t)(p.zrep > 1 ? p.zrep : bo) * M * R * 8, 256);
  const size_t obytes = (size_t)(p.ks2 - 1) * bo * M * Q * 8;
  if (ybytes + zbytes + obytes > decode2_region_bytes()) return d2_bail(__LINE__);
  p.ypart = reinterpret_cast<unsigned long long*>(region);
  p.zt = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes);
  p.opart = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes + zbytes);
  p.epoch_word = epoch_word; p.arrive_word = arrive_word; p.err_word = err_word; p.spin_limit = spin_limit_now();

  int grid = p.items1 + p.items2;
  if (grid > resident) grid = resident;
  if (grid < p.items1) grid = p.items1;
  if (grid < p.items2) grid = p.items2;
  if (grid < p.itemsM) grid = p.itemsM;
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, 0, st);
  if (e != hipSuccess) { set_error("decode2: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

// Matrix-core variant of the launch (any M <= 16).
int decode2m_blast_launch(const StreamBlastArgs& a, void* region, unsigned* epoch_word, unsigned* arrive_word,
                          unsigned* err_word, hipStream_t st) {
  const int bo = a.bo > 0 ? a.bo : a.b;
  const int P = a.in_f / a.b, Q = a.out_f / bo, R = a.r, b = a.b, M = a.M;
  if (a.wbits != 16 && !((a.wbits == 8 || a.wbits == 4) && a.u_layout == BLR_U_RQ && a.u_scales && a.v_scales)) return d2_bail(__LINE__);   // two-byte weights, or codes stored (k, n)
  void* fn = a.wbits == 8 ? (a.dtype == BLR_F16 ? (void*)decode2m_kernel<f16, 8> : (void*)decode2m_kernel<bf16, 8>)
           : a.wbits == 4 ? (a.dtype == BLR_F16 ? (void*)decode2m_kernel<f16, 4> : (void*)decode2m_kernel<bf16, 4>)
                          : (a.dtype == BLR_F16 ? (void*)decode2m_kernel<f16, 16> : (void*)decode2m_kernel<bf16, 16>);
  static std::mutex mu;
  static std::map<void*, int> occ_cache;
  int occ = 0;
  {
    std::lock_guard<std::mutex> lk(mu);
    auto it = occ_cache.find(fn);
    if (it != occ_cache.end()) occ = it->second;
    else {
      hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, 256, 0);
      if (e != hipSuccess || occ < 1) { (void)hipGetLastError(); set_error("decode2m: occupancy query failed"); return BLR_ERR_LAUNCH; }
      occ_cache[fn] = occ;
    }
  }
  const int cus = device_cus() > 0 ? device_cus() : 256;
  const int resident = (occ < 2 ? occ : 2) * cus;
  if (R % 4) return d2_bail(__LINE__);

  Decode2Params p = {};
  p.x = a.x; p.ldx = a.ldx; p.V = a.V; p.U = a.U; p.S = a.S; p.out = a.out; p.ldo = a.ldo;
  p.u_scales = (const f16*)a.u_scales; p.v_scales = (const f16*)a.v_scales;
  p.M = M; p.b = b; p.bo = bo; p.P = P; p.R = R; p.Q = Q;
  p.perm_per = a.perm_per; p.o_bs = a.out_ns ? a.out_bs : Q; p.o_ns = a.out_ns ? a.out_ns : 1;
  if (a.s_layout == BLR_S_JIR) { p.s_sj = (int64_t)b * R; p.s_si = R; p.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { p.s_sr = (int64_t)b * b; p.s_si = b; p.s_sj = 1; }
  else { p.s_si = (int64_t)b * R; p.s_sj = R; p.s_sr = 1; }
  {
    const int nch = (R + 127) / 128, base = b * nch;
    if (base > resident) return d2_bail(__LINE__);
    int ks = (P + DM_ROWS - 1) / DM_ROWS;       // one batch per slice if the grid allows
    if (ks > resident / base) ks = resident / base;
    if (ks > 4) ks = 4;
    if (ks < 1) ks = 1;
    int kc = (P + ks - 1) / ks;
    kc = (kc + 7) / 8 * 8;
    if (kc > DM_KMAX) kc = DM_KMAX;
    ks = (P + kc - 1) / kc;
    if (ks > 4 || base * ks > resident) return d2_bail(__LINE__);
    p.lpr1_log2 = 4; p.nch1 = nch; p.ks1 = ks; p.kc1 = kc; p.items1 = base * ks;
    // a slice of x may be fetched in 16-byte pieces if every piece is aligned and inside the row
    p.x_vec = aligned(a.x, 16) && a.ldx % 8 == 0 && P % 8 == 0 && kc % 8 == 0;
  }
  {
    constexpr int ks_cap = 4;
    const int nch = (Q + 127) / 128, base = bo * nch;
    if (base > resident) return d2_bail(__LINE__);
    // BLAST proper (b output blocks): no k split of stage 2 - handing partial outputs of up to 16 rows between workgroups
    // costs more than the shorter slabs save (measured at every M from 5 to 16); low rank and Monarch keep the split
    const bool no_split = bo == b && bo > 1 && a.perm_per == 0;
    int ks = no_split ? 1 : resident / base;
    if (ks > ks_cap) ks = ks_cap;
    if (ks > 4) ks = 4;
    if (ks > resident / base) ks = resident / base;
    if (ks < 1) ks = 1;
    int kc = (R + ks - 1) / ks;
    kc = (kc + DM_ROWS - 1) / DM_ROWS * DM_ROWS;
    if (kc > DM_KMAX) kc = DM_KMAX;
    ks = (R + kc - 1) / kc;
    if (ks > 4 || base * ks > resident) return d2_bail(__LINE__);
    int pfn = (kc + DM_ROWS - 1) / DM_ROWS * 8;
    const int pf_cap = a.wbits == 16 ? DM_PF : 2 * DM_PF;    // narrower loads of codes: twice as many in no more registers
    if (pfn > pf_cap) pfn = pf_cap;
    p.lpr2_log2 = 4; p.nch2 = nch; p.ks2 = ks; p.kc2 = kc; p.items2 = base * ks; p.pfn = pfn;
    p.kpad2 = (kc + DM_ROWS - 1) / DM_ROWS * DM_ROWS;
    p.u_nk = a.u_layout == BLR_U_QR;
  }
  {
    p.zrep = bo == 1 ? 16 : 1;
    int bp2 = 2;                                   // at least two ranks per mix thread row: z goes out in pairs
    while (bp2 < b || bp2 < bo || bp2 < p.zrep) bp2 <<= 1;
    if (bp2 > 128) return d2_bail(__LINE__);
    const int rch = 256 / bp2;
    p.rch_log2 = ilog2(rch);
    p.itemsM = ((R + rch - 1) / rch) * ((M + DM_MC - 1) / DM_MC);
    if (p.itemsM > resident) return d2_bail(__LINE__);
    p.pf_depth = 4;
  }
  const size_t ybytes = align_up((size_t)p.ks1 * b * M * R * 8, 256), zbytes = align_up((size_t)(p.zrep > 1 ? p.zrep : bo) * M * (R / 2) * 8, 256);
  const size_t obytes = (size_t)(p.ks2 - 1) * bo * M * Q * 8;
  if (ybytes + zbytes + obytes > decode2_region_bytes()) return d2_bail(__LINE__);
  p.ypart = reinterpret_cast<unsigned long long*>(region);
  p.zt = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes);
  p.opart = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(region) + ybytes + zbytes);
  p.epoch_word = epoch_word; p.arrive_word = arrive_word; p.err_word = err_word; p.spin_limit = spin_limit_now();
  int grid = p.items1 + p.items2;
  if (grid > resident) grid = resident;
  if (grid < p.items1) grid = p.items1;
  if (grid < p.items2) grid = p.items2;
  if (grid < p.itemsM) grid = p.itemsM;
  void* args[] = {&p};
  hipError_t e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, 0, st);
  if (e != hipSuccess) { set_error("decode2m: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

// Batched C[bt] = A[bt] B[bt] at up to 16 rows through dense_slab_kernel; B (K, N) row-major with row stride ldb.
// part: room for max_slices * batch * M * N floats (may be null with max_slices <= 1: the reduction is then not cut, which
// limits K to one slab).  Returns BLR_OK, a negative status, or 1 when the call is not for this kernel.
int slab_gemm_launch(const void* A, int64_t lda, int64_t sA, const void* B, int64_t ldb, int64_t sB, void* C, int64_t ldc, int64_t sC,
                     int M, int N, int K, int batch, int dtype, float* part, int max_slices, hipStream_t st) {
  if (!option_value(OPT_DENSE_SLAB, 1) || M < 1 || M > 16) return 1;
  if (dtype != BLR_F16 && dtype != BLR_BF16) return 1;
  if (N % 8 || ldb % 8 || sB % 8 || !aligned(B, 16) || (int64_t)K * ldb * 2 >= (1ll << 31)) return d2_bail(__LINE__);   // 16-byte pieces of a row, 32-bit buffer offsets
  if (!part || max_slices < 1) max_slices = 1;
  const int cus = device_cus() > 0 ? device_cus() : 256;
  const int nch = (N + 127) / 128;
  const int64_t base = (int64_t)nch * batch;
  // Slices: one workgroup per compute unit if its slab then fits the four register batches (512 rows: the whole slab is
  // requested at once and the partial sums stay few), otherwise two per compute unit.
  int ks = 1, kc = K;
  for (int per_cu = 1; per_cu <= 2; ++per_cu) {
    ks = (int)(((int64_t)per_cu * cus + base - 1) / base);   // enough slices to give every compute unit its workgroups
    if (ks > max_slices) ks = max_slices;
    if (ks > (K + DM_ROWS - 1) / DM_ROWS) ks = (K + DM_ROWS - 1) / DM_ROWS;
    if (ks < 1) ks = 1;
    kc = ((K + ks - 1) / ks + DM_ROWS - 1) / DM_ROWS * DM_ROWS;
    const bool fits = kc <= DM_PF / 8 * DM_ROWS;
    if (kc > DM_KMAX) kc = DM_KMAX;
    ks = (K + kc - 1) / kc;
    if (fits) break;
  }
  if (ks > max_slices) return d2_bail(__LINE__);
  if (base * ks >= (1ll << 31)) return d2_bail(__LINE__);
  DenseSlabParams p = {};
  p.x = A; p.ldx = lda; p.W = B; p.out = C; p.ldo = ldc; p.part = part;
  p.sx = sA; p.sw = sB; p.so = sC; p.ldw = ldb;
  p.M = M; p.K = K; p.N = N; p.nch = nch; p.ks = ks; p.kc = kc; p.batch = batch;
  p.x_vec = aligned(A, 16) && lda % 8 == 0 && sA % 8 == 0 && K % 8 == 0;
  const unsigned grid = (unsigned)(base * ks);
  if (dtype == BLR_F16) hipLaunchKernelGGL(dense_slab_kernel<f16>, dim3(grid), dim3(256), 0, st, p);
  else hipLaunchKernelGGL(dense_slab_kernel<bf16>, dim3(grid), dim3(256), 0, st, p);
  if (ks > 1) {
    const unsigned blocks = (unsigned)(((int64_t)batch * M * N + 255) / 256);
    if (dtype == BLR_F16) hipLaunchKernelGGL(dense_slab_reduce_kernel<f16>, dim3(blocks), dim3(256), 0, st, part, (f16*)C, ldc, sC, M, N, ks, batch);
    else hipLaunchKernelGGL(dense_slab_reduce_kernel<bf16>, dim3(blocks), dim3(256), 0, st, part, (bf16*)C, ldc, sC, M, N, ks, batch);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("dense_slab: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

int dense_slab_launch(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo, int M, int K, int N, int dtype,
                      float* part, int max_slices, hipStream_t st) {
  return slab_gemm_launch(x, ldx, 0, W, N, 0, out, ldo, 0, M, N, K, 1, dtype, part, max_slices, st);
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace2(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace2), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

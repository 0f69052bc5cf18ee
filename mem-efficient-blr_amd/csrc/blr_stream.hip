// Streaming engine for decode-sized calls (M <= 16): every weight byte is read exactly once, at
// full width, by a persistent grid that stays resident for the whole call.
//
// A call is a short list of phases executed by one kernel, separated by grid-wide barriers
// (or, in "split" mode, by one launch per phase):
//   KN  : skinny product against (k, n)-ordered weights (n contiguous).  A workgroup streams a
//         [k-chunk] x [n-chunk] slab with 16-byte loads, lanes own 8 consecutive n, row slots
//         split k; partial sums over k-chunks go to slots and the last workgroup to finish a
//         column chunk adds them in a fixed order (deterministic, no float atomics).
//   NK  : skinny product against (n, k)-ordered weights (k contiguous).  A wave owns 16 weight
//         rows and feeds them straight from global memory into v_mfma_f32_16x16x32 as the B
//         operand; the (<= 16) activation rows sit in LDS as the A operand.
//   MIX : BLAST rank-space mix  Z_i = sum_j S_ij * Y_j  as its own phase (M > 2); for M <= 2 the
//         consumer phase recomputes the slice of Z it needs while staging its activations.
// Intermediates (Y, Z, low-rank z, Monarch out1, split-k partials) are fp32 in the caller's
// workspace.  They are written and read with device-scope accesses, which bypass the per-XCD L2,
// so that no cache write-back or invalidate is needed at a barrier: a workgroup only has to wait
// for its own stores to be acknowledged before it reports in.
// The first batch of the last phase's weight loads is issued before anything else, so HBM is busy
// while the earlier phases and barriers run.
#include <cstdlib>
#include <map>
#include <mutex>
#include <utility>
#include "blr_common.h"
#include "blr_decode.h"

namespace blr {

enum { PH_NONE = 0, PH_KN = 1, PH_NK = 2, PH_MIX = 3 };
enum { A_X = 0, A_F32 = 1, A_MIX = 2, A_Z = 3 };      // A_Z: like A_F32, read from the current Z accumulation buffer
enum { E_F32 = 0, E_OUT = 1, E_ZATOM = 2 };            // E_ZATOM: BLAST stage 1 adds S_ij * y straight into Z_i (atomics)

constexpr int AS_FLOATS = 4096;  // KN: fp32 activation floats staged in LDS (MT * k-chunk <= this)
constexpr int NC_MAX = 512;      // widest KN column chunk (64 lanes x 8)
constexpr int RED_MG = 2;        // activation rows reduced across waves per pass
constexpr int UNR = 8;           // 16-byte weight loads in flight per lane
constexpr int KSPLIT_MAX = 64;
constexpr unsigned SPIN_LIMIT = 2000000u;

#ifdef BLR_TRACE
__device__ unsigned long long g_trace[1024 * 16];
#define TR(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) g_trace[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TR(i) do {} while (0)
#endif

struct PhaseDesc {
  int kind, wbits;
  const void* W; int64_t w_bs, ldw;         // element (code) units
  int batch, K, N;
  int lpr_log2, kc, ksplit, nchunks;        // KN tiling
  int nk_split_k;                           // NK: the 4 waves of a workgroup split K instead of rows
  int kn_mfma;                              // KN: matrix-core variant (lanes transpose 8x8 blocks in registers)
  int amode; const void* a; int64_t lda, a_bs;
  int emode; void* o; int64_t ldo, o_bs, o_ns;
  int perm_per;                             // > 0: Monarch scatter on E_F32
  const f16* o_scales;                      // per (bt, n) output scale or null
  float* part; unsigned* counters;
  const float* Y; const void* S; int64_t s_si, s_sj, s_sr; int b, R; const f16* v_scales;   // MIX / A_MIX
  int vec_ok;
};

struct StreamParams {
  PhaseDesc ph[3];
  int nph, M, use_barrier;
  int zatom, first, finish;                  // Z accumulation in use; launch holds the first / the last phase of the call
  float* zbuf[2]; unsigned zextent;          // two fixed-place Z buffers (ping-pong between calls), floats used by this call
  unsigned* ctrl;                           // barrier shards / finished counters / error word (see grid_barrier)
  unsigned spin_limit;                      // polls after which the barrier gives up
};

// ---- device-scope accessors for data exchanged between workgroups ----------------------------------
__device__ __forceinline__ float ld_dev(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// Wait until every store this wave issued has been acknowledged.
__device__ __forceinline__ void drain_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---- grid barrier ---------------------------------------------------------------------------
// All workgroups of the launch are resident (the host sizes the grid from the occupancy query),
// so every arrival is eventually seen.  Arrivals are spread over BAR_SHARDS counters on separate
// cache lines (same-address atomics serialise at the memory side); a waiting wave reads all shards
// with one vector load.  The wait is bounded: on expiry the error word is set and the workgroup
// carries on, so the grid always drains.
constexpr int BAR_SHARDS = 16;
constexpr int BAR_STRIDE = 64;                    // uint32 words between shard counters (256 bytes)
constexpr int BAR_DONE = BAR_SHARDS * BAR_STRIDE; // per-shard "finished" counters follow the arrival counters
constexpr int BAR_ERR = 2 * BAR_SHARDS * BAR_STRIDE;
constexpr int BAR_GDONE = BAR_ERR + 64;           // shards that have fully finished (end-of-call bookkeeping)
constexpr int Z_PARITY = BAR_ERR + 128;           // which Z buffer the current call accumulates into
constexpr int Z_DIRTY = BAR_ERR + 192;            // [2] floats of each Z buffer that are not known to be zero
constexpr int D2_EPOCH = BAR_ERR + 256;           // call counter of the two-stage decode kernel
constexpr int D2_ARRIVE = BAR_ERR + 320;          // its check-in counter

__device__ __forceinline__ unsigned shard_population(int shard) {   // workgroups whose index maps to `shard`
  return ((unsigned)gridDim.x + BAR_SHARDS - 1 - shard) / BAR_SHARDS;
}

__device__ __forceinline__ void grid_barrier(unsigned* ctrl, unsigned nth, unsigned spin_limit) {
  drain_stores();
  __syncthreads();
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    if (lane == 0)
      __hip_atomic_fetch_add(&ctrl[(blockIdx.x % BAR_SHARDS) * BAR_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int s = lane % BAR_SHARDS;
    const unsigned target = nth * shard_population(s);
    unsigned spins = 0;
    while (true) {
      unsigned v = __hip_atomic_load(&ctrl[s * BAR_STRIDE], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__all(v >= target)) break;
      __builtin_amdgcn_s_sleep(1);
      if (++spins > spin_limit) {
        if (lane == 0) __hip_atomic_store(&ctrl[BAR_ERR], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
  }
  __syncthreads();
}

// End-of-call bookkeeping.  The last workgroup of each shard to finish re-arms that shard; the last
// shard to do so flips the Z ping-pong: the buffer this call accumulated into becomes "dirty", the
// other one (zeroed by this call) becomes the next call's accumulator.
__device__ __forceinline__ void call_finish(const StreamParams& p, unsigned parity) {
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned* ctrl = p.ctrl;
    const int s = blockIdx.x % BAR_SHARDS;
    unsigned old = __hip_atomic_fetch_add(&ctrl[BAR_DONE + s * BAR_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == shard_population(s) - 1) {
      __hip_atomic_store(&ctrl[s * BAR_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&ctrl[BAR_DONE + s * BAR_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (p.zatom && p.finish) {
        const unsigned live = gridDim.x < (unsigned)BAR_SHARDS ? gridDim.x : (unsigned)BAR_SHARDS;
        unsigned g = __hip_atomic_fetch_add(&ctrl[BAR_GDONE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (g == live - 1) {                        // every workgroup of the call is done
          __hip_atomic_store(&ctrl[BAR_GDONE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(&ctrl[Z_DIRTY + parity], p.zextent, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(&ctrl[Z_DIRTY + (parity ^ 1u)], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(&ctrl[Z_PARITY], parity ^ 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
}

// 16-byte device-scope load (sc0 sc1: served from memory, not from this XCD's possibly stale L2).
__device__ __forceinline__ f32x4 ld_dev4(const float* base, uint32_t byte_off) {
  __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, 0x7fffffff, 0x00020000);
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 17));
}

// ---- weight fetch: 8 consecutive elements ------------------------------------------------------
// Raw register image of 8 consecutive weights: 16 bytes of f16/bf16, 8 bytes of int8 codes or
// 4 bytes of int4 codes.  Loads are kept raw so that a whole batch of them can be issued
// back to back before the first conversion.
template <int WB> struct Raw8;
template <> struct Raw8<16> { u32x4 v; };
template <> struct Raw8<8> { u32x2 v; };
template <> struct Raw8<4> { uint32_t v; };

template <int WB>
__device__ __forceinline__ Raw8<WB> load_raw8(const void* W, int64_t eoff) {
  Raw8<WB> r;
  if (WB == 16) r.v = __builtin_nontemporal_load(reinterpret_cast<const decltype(r.v)*>(reinterpret_cast<const uint16_t*>(W) + eoff));
  else if (WB == 8) r.v = __builtin_nontemporal_load(reinterpret_cast<const decltype(r.v)*>(reinterpret_cast<const uint8_t*>(W) + eoff));
  else r.v = __builtin_nontemporal_load(reinterpret_cast<const decltype(r.v)*>(reinterpret_cast<const uint8_t*>(W) + (eoff >> 1)));
  return r;
}

template <typename T>
__device__ __forceinline__ void raw_to_f32(const Raw8<16>& r, float (&w)[8]) {
  typename TypeTraits<T>::vec8 v = __builtin_bit_cast(typename TypeTraits<T>::vec8, r.v);
#pragma unroll
  for (int e = 0; e < 8; ++e) w[e] = TypeTraits<T>::to_f32(v[e]);
}
template <typename T>
__device__ __forceinline__ void raw_to_f32(const Raw8<8>& r, float (&w)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) w[e] = (float)(int8_t)((r.v[e >> 2] >> ((e & 3) * 8)) & 0xFF);
}
template <typename T>
__device__ __forceinline__ void raw_to_f32(const Raw8<4>& r, float (&w)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) w[e] = (float)(((int32_t)(r.v << (28 - 4 * e))) >> 28);
}

// Element-wise fetch for rows that are not 16-byte friendly (tiny or odd shapes; f16/bf16 only).
template <typename T>
__device__ __forceinline__ void fetch8_scalar(const void* W, int64_t eoff, int nvalid, float (&w)[8]) {
  const T* p = reinterpret_cast<const T*>(W) + eoff;
#pragma unroll
  for (int e = 0; e < 8; ++e) w[e] = (e < nvalid) ? TypeTraits<T>::to_f32(p[e]) : 0.0f;
}

template <typename T>
__device__ __forceinline__ void emit(const PhaseDesc& d, int M, int bt, int m, int n, float v, float* zcur = nullptr) {
  if (d.o_scales) v *= (float)d.o_scales[(int64_t)bt * d.N + n];
  if (d.emode == E_OUT) {
    reinterpret_cast<T*>(d.o)[(int64_t)m * d.ldo + (int64_t)bt * d.o_bs + (int64_t)n * d.o_ns] = TypeTraits<T>::from_f32(v);
  } else if (d.emode == E_ZATOM) {
    // v = Y[j = bt][m][r = n]: its contribution S(i, j, r) * vscale(j, r) * v goes to every Z_i
    const T* S = reinterpret_cast<const T*>(d.S);
    if (d.v_scales) v *= (float)d.v_scales[(int64_t)bt * d.R + n];
    for (int i = 0; i < d.b; ++i) {
      float sx = TypeTraits<T>::to_f32(S[(int64_t)i * d.s_si + (int64_t)bt * d.s_sj + (int64_t)n * d.s_sr]);
      __hip_atomic_fetch_add(&zcur[((int64_t)i * M + m) * d.R + n], sx * v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    float* o = reinterpret_cast<float*>(d.o);
    if (d.perm_per > 0) {
      int dst = n / d.perm_per, j = n - dst * d.perm_per;
      st_dev(&o[((int64_t)dst * M + m) * d.ldo + (int64_t)bt * d.perm_per + j], v);
    } else {
      st_dev(&o[((int64_t)bt * M + m) * d.ldo + n], v);
    }
  }
}

// One activation value A[bt][m][k] of a phase.
template <typename T>
__device__ __forceinline__ float act_load(const PhaseDesc& d, int M, int bt, int m, int k, const float* zcur = nullptr) {
  if (d.amode == A_Z) return ld_dev(&zcur[((int64_t)bt * M + m) * d.K + k]);
  if (d.amode == A_X) return TypeTraits<T>::to_f32(reinterpret_cast<const T*>(d.a)[(int64_t)m * d.lda + (int64_t)bt * d.a_bs + k]);
  if (d.amode == A_F32) return ld_dev(&reinterpret_cast<const float*>(d.a)[((int64_t)bt * M + m) * d.K + k]);
  // A_MIX: Z[i = bt][m][r = k] = sum_j S(i, j, r) * vscale(j, r) * Y[j][m][r]; loads first, then the sum
  const T* S = reinterpret_cast<const T*>(d.S);
  float acc = 0.0f;
  for (int j0 = 0; j0 < d.b; j0 += 16) {
    float yv[16], sv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int j = j0 + u;
      const bool ok = j < d.b;
      yv[u] = ok ? ld_dev(&d.Y[((int64_t)j * M + m) * d.R + k]) : 0.0f;
      sv[u] = ok ? TypeTraits<T>::to_f32(S[(int64_t)bt * d.s_si + (int64_t)j * d.s_sj + (int64_t)k * d.s_sr]) : 0.0f;
      if (ok && d.v_scales) sv[u] *= (float)d.v_scales[(int64_t)j * d.R + k];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) acc = fmaf(sv[u], yv[u], acc);
  }
  return acc;
}

// Split-k epilogue of a KN item: once this workgroup's partial sums are device-visible it checks
// in on the column chunk's counter; the last one to do so adds all slots in a fixed order and emits.
template <typename T>
__device__ __forceinline__ void kn_splitk_finish(const PhaseDesc& d, int M, int bt, int nc, int n0, int NC, float* red,
                                                 float* zcur, int trb) {
  __shared__ int s_last;
  const int tid = threadIdx.x;
  if (d.ksplit <= 1) return;
  drain_stores();                                  // this workgroup's partial sums are device-visible
  __syncthreads();
  if (tid == 0) {
    unsigned old = __hip_atomic_fetch_add(&d.counters[bt * d.nchunks + nc], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == (unsigned)(d.ksplit - 1));
  }
  __syncthreads();
  TR(trb + 4);
  if (!s_last) return;                             // (uniform over the workgroup)
  const int64_t slot = (int64_t)d.batch * M * d.N;
  if ((d.N & 3) == 0 && slot * d.ksplit * 4 < 0x7fffffffLL) {
    // All 256 threads: thread (vc, sg) adds slots sg, sg+G, ... of four columns, then the G
    // groups are added in order through LDS.  One or two rounds of 16-byte loads in total.
    const int vcols = NC >> 2;
    const int G = 256 / vcols;
    const int vc = tid % vcols, sg = tid / vcols;
    f32x4* red4 = reinterpret_cast<f32x4*>(red);
    for (int m = 0; m < M; ++m) {
      f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      const int gn = n0 + vc * 4;
      if (sg < G && gn < d.N) {
        const uint32_t off0 = (uint32_t)((((int64_t)bt * M + m) * d.N + gn) * 4);
        int sidx = sg;
        for (; sidx + 7 * G < d.ksplit; sidx += 8 * G) {
          f32x4 t[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) t[u] = ld_dev4(d.part, off0 + (uint32_t)((sidx + u * G) * slot * 4));
#pragma unroll
          for (int u = 0; u < 8; ++u) v += t[u];
        }
        for (; sidx < d.ksplit; sidx += G) v += ld_dev4(d.part, off0 + (uint32_t)(sidx * slot * 4));
      }
      __syncthreads();
      if (sg < G) red4[sg * vcols + vc] = v;
      __syncthreads();
      if (tid < vcols && gn < d.N) {
        f32x4 t = red4[tid];
        for (int g = 1; g < G; ++g) t += red4[g * vcols + tid];
#pragma unroll
        for (int e = 0; e < 4; ++e) emit<T>(d, M, bt, m, gn + e, t[e], zcur);
      }
    }
  } else {
    for (int idx = tid; idx < NC * M; idx += 256) {
      int m = idx / NC, col = idx - m * NC;
      int gn = n0 + col;
      if (gn >= d.N) continue;
      const float* p0 = &d.part[((int64_t)bt * M + m) * d.N + gn];
      float v = 0.0f;
      for (int sidx = 0; sidx < d.ksplit; ++sidx) v += ld_dev(p0 + sidx * slot);
      emit<T>(d, M, bt, m, gn, v, zcur);
    }
  }
  if (tid == 0) __hip_atomic_store(&d.counters[bt * d.nchunks + nc], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- KN phase -----------------------------------------------------------------------------------
struct KnItem {
  int nc, ks, bt, k0, kc, n0, n;
  bool col_ok;
  int64_t wbase;
};
__device__ __forceinline__ KnItem kn_item(const PhaseDesc& d, int item, int cv) {
  KnItem it;
  it.nc = item % d.nchunks;
  const int t2 = item / d.nchunks;
  it.ks = t2 % d.ksplit; it.bt = t2 / d.ksplit;
  it.k0 = it.ks * d.kc; it.kc = min(d.kc, d.K - it.k0);
  it.n0 = it.nc * (8 << d.lpr_log2);
  it.n = it.n0 + cv * 8;
  it.col_ok = it.n < d.N;
  it.wbase = (int64_t)it.bt * d.w_bs + (int64_t)it.k0 * d.ldw + (it.col_ok ? it.n : 0);
  return it;
}

template <typename T, int MT, int WB, bool VEC>
__device__ __forceinline__ void phase_kn(const PhaseDesc& d, int M, float* smem, int trb, float* zcur) {
  constexpr int KC_LD = AS_FLOATS / MT;            // row stride of the staged activations
  float* a_s = smem;                               // [MT][KC_LD]
  float* red = smem + AS_FLOATS;                   // [4 waves][RED_MG][NC_MAX]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lpr = 1 << d.lpr_log2, rpp = 256 >> d.lpr_log2;
  const int cv = tid & (lpr - 1), rs = tid >> d.lpr_log2;
  const int NC = lpr * 8;
  const int total = d.batch * d.ksplit * d.nchunks;
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const KnItem it = kn_item(d, item, cv);
    const int bt = it.bt, kc = it.kc, n0 = it.n0;

    // Weight rows do not depend on the activations: get the first batch in flight before staging.
    int kk = rs;
    Raw8<WB> raw[UNR];
    bool have_raw = false;
    // Whole chunk inside the matrix and room for one batch of zero activations behind the slice: every batch is full and
    // every load unconditional (rows past the slice are fetched from its last row and multiplied by zeros) - a load under
    // a condition makes the compiler wait for all loads in flight at every use.
    const bool fast = VEC && n0 + NC <= d.N && kc + UNR * rpp <= KC_LD;
    if (fast) {
#pragma unroll
      for (int u = 0; u < UNR; ++u) raw[u] = load_raw8<WB>(d.W, it.wbase + (int64_t)min(kk + u * rpp, kc - 1) * d.ldw);
    } else if (VEC && it.col_ok && kk + (UNR - 1) * rpp < kc) {
#pragma unroll
      for (int u = 0; u < UNR; ++u) raw[u] = load_raw8<WB>(d.W, it.wbase + (int64_t)(kk + u * rpp) * d.ldw);
      have_raw = true;
    }
    __syncthreads();
    if ((d.amode == A_F32 || d.amode == A_Z) && ((d.K | it.k0 | kc) & 3) == 0) {       // 16-byte device-scope loads
      const int kq = kc >> 2;
      for (int idx = tid; idx < MT * kq; idx += 256) {
        int m = idx / kq, ka = (idx - m * kq) * 4;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (m < M) v = ld_dev4(d.amode == A_Z ? zcur : reinterpret_cast<const float*>(d.a), (uint32_t)((((int64_t)bt * M + m) * d.K + it.k0 + ka) * 4));
        *reinterpret_cast<f32x4*>(&a_s[m * KC_LD + ka]) = v;
      }
    } else {
      for (int idx = tid; idx < MT * kc; idx += 256) {
        int m = idx / kc, ka = idx - m * kc;
        a_s[m * KC_LD + ka] = (m < M) ? act_load<T>(d, M, bt, m, it.k0 + ka, zcur) : 0.0f;
      }
    }
    if (fast) {
      for (int idx = tid; idx < MT * UNR * rpp; idx += 256) {
        const int m = idx / (UNR * rpp), ka = idx - m * (UNR * rpp);
        a_s[m * KC_LD + kc + ka] = 0.0f;
      }
    }
    __syncthreads();
    TR(trb + 1);

    float acc[MT][8];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[m][e] = 0.0f;
    if (fast) {
      for (int kcur = kk; kcur < kc; kcur += UNR * rpp) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          float w[8];
          raw_to_f32<T>(raw[u], w);
          raw[u] = load_raw8<WB>(d.W, it.wbase + (int64_t)min(kcur + (UNR + u) * rpp, kc - 1) * d.ldw);   // refill the slot right away
          const int k = kcur + u * rpp;
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const float a = a_s[m * KC_LD + k];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[m][e] = fmaf(a, w[e], acc[m][e]);
          }
        }
      }
    } else if (it.col_ok) {
      if (VEC) {
        while (have_raw) {
          const int kcur = kk;
          kk += UNR * rpp;
          const bool more = kk + (UNR - 1) * rpp < kc;
#pragma unroll
          for (int u = 0; u < UNR; ++u) {
            float w[8];
            raw_to_f32<T>(raw[u], w);
            // the slot is free again: refill it right away so UNR loads stay in flight
            if (more) raw[u] = load_raw8<WB>(d.W, it.wbase + (int64_t)(kk + u * rpp) * d.ldw);
            const int k = kcur + u * rpp;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              float a = a_s[m * KC_LD + k];
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[m][e] = fmaf(a, w[e], acc[m][e]);
            }
          }
          have_raw = more;
        }
        for (; kk < kc; kk += rpp) {               // leftover rows
          float w[8];
          raw_to_f32<T>(load_raw8<WB>(d.W, it.wbase + (int64_t)kk * d.ldw), w);
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float a = a_s[m * KC_LD + kk];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[m][e] = fmaf(a, w[e], acc[m][e]);
          }
        }
      } else {
        const int nvalid = min(8, d.N - it.n);
        for (; kk < kc; kk += rpp) {
          float w[8];
          fetch8_scalar<T>(d.W, it.wbase + (int64_t)kk * d.ldw, nvalid, w);
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float a = a_s[m * KC_LD + kk];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[m][e] = fmaf(a, w[e], acc[m][e]);
          }
        }
      }
    }
    TR(trb + 2);
    // row slots inside a wave
    for (int o = lpr; o < 64; o <<= 1) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[m][e] += __shfl_xor(acc[m][e], o, 64);
    }
    // across waves, RED_MG activation rows at a time
#pragma unroll
    for (int mg = 0; mg < MT; mg += RED_MG) {
      __syncthreads();
      if (lane < lpr) {
#pragma unroll
        for (int mm = 0; mm < RED_MG; ++mm) {
          if (mg + mm < MT) {
#pragma unroll
            for (int e = 0; e < 8; ++e) red[(wave * RED_MG + mm) * NC_MAX + cv * 8 + e] = acc[mg + mm < MT ? mg + mm : 0][e];
          }
        }
      }
      __syncthreads();
      for (int col = tid; col < NC; col += 256) {
        int gn = n0 + col;
        if (gn >= d.N) continue;
        for (int mm = 0; mm < RED_MG; ++mm) {
          int m = mg + mm;
          if (m >= M || m >= MT) break;
          float v = red[(0 * RED_MG + mm) * NC_MAX + col] + red[(1 * RED_MG + mm) * NC_MAX + col] +
                    red[(2 * RED_MG + mm) * NC_MAX + col] + red[(3 * RED_MG + mm) * NC_MAX + col];
          if (d.ksplit == 1) emit<T>(d, M, bt, m, gn, v, zcur);
          else st_dev(&d.part[(((int64_t)it.ks * d.batch + bt) * M + m) * d.N + gn], v);
        }
      }
    }
    TR(trb + 3);
    kn_splitk_finish<T>(d, M, bt, it.nc, n0, NC, red, zcur, trb);
  }
}

// ---- KN phase on the matrix cores (M up to 16 at the cost of M = 1) ------------------------------------
// Column chunk of 128 (16 lanes x 8), 16 row slots of 8 consecutive rows: one batch of eight
// 16-byte loads per lane covers 128 rows x 128 columns.  Each lane transposes its 8x8 block in
// registers (v_perm) into eight B fragments of v_mfma_f32_16x16x32 - fragment e holds column
// 8*cv + e for the lane's 8 rows - and the activations, staged in LDS as [16][k], are the A
// fragment.  A wave contracts its own 32 rows per batch; the four waves are added through LDS.
constexpr int KNM_KC_MAX = 2048;                 // 16 x (2048 + 8) two-byte activations: 66 KB of LDS, two workgroups per CU

template <typename T>
__device__ __forceinline__ void phase_kn_mfma(const PhaseDesc& d, int M, float* smem, int trb, float* zcur) {
  using V8 = typename TypeTraits<T>::vec8;
  T* a_s = reinterpret_cast<T*>(smem);              // [16][ka_ld]
  float* red = smem;                               // [4 waves][4 fragments][64 lanes][4]; reuses the staging area once the products are done
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cv = lane & 15, kg = lane >> 4, rs = wave * 4 + kg;
  const int NC = 128;
  const int total = d.batch * d.ksplit * d.nchunks;
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const KnItem it = kn_item(d, item, cv);
    const int bt = it.bt, kc = it.kc, n0 = it.n0;
    const int kcp = (kc + 127) / 128 * 128;
    const int ka_ld = kcp + 8;
    u32x4 raw[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) raw[u] = load_raw8<16>(d.W, it.wbase + (int64_t)min(rs * 8 + u, kc - 1) * d.ldw).v;
    __syncthreads();
    if ((d.amode == A_F32 || d.amode == A_Z) && ((d.K | it.k0 | kc) & 3) == 0) {
      const int kq = kcp >> 2;
      for (int idx = tid; idx < 16 * kq; idx += 256) {
        int m = idx / kq, ka = (idx - m * kq) * 4;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (m < M && ka < kc) v = ld_dev4(d.amode == A_Z ? zcur : reinterpret_cast<const float*>(d.a), (uint32_t)((((int64_t)bt * M + m) * d.K + it.k0 + ka) * 4));
#pragma unroll
        for (int e = 0; e < 4; ++e) a_s[m * ka_ld + ka + e] = TypeTraits<T>::from_f32(v[e]);
      }
    } else if (d.amode == A_X && ((d.lda | d.a_bs | it.k0 | kc) & 7) == 0 && (reinterpret_cast<uintptr_t>(d.a) & 15) == 0) {
      // activations straight from x in 16-byte pieces (they already have the element type of the A fragment)
      const int pieces = kcp >> 3;
      const T* xp = reinterpret_cast<const T*>(d.a);
      for (int idx = tid; idx < 16 * pieces; idx += 256) {
        int m = idx / pieces, ka = (idx - m * pieces) * 8;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (m < M && ka < kc) v = *reinterpret_cast<const u32x4*>(&xp[(int64_t)m * d.lda + (int64_t)bt * d.a_bs + it.k0 + ka]);
        *reinterpret_cast<u32x4*>(&a_s[m * ka_ld + ka]) = v;
      }
    } else {
      for (int idx = tid; idx < 16 * kcp; idx += 256) {
        int m = idx / kcp, ka = idx - m * kcp;
        a_s[m * ka_ld + ka] = TypeTraits<T>::from_f32((m < M && ka < kc) ? act_load<T>(d, M, bt, m, it.k0 + ka, zcur) : 0.0f);
      }
    }
    __syncthreads();
    TR(trb + 1);
    f32x4 acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int kcur = 0; kcur < kcp; kcur += 128) {
      u32x4 cur[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) cur[u] = raw[u];
      if (kcur + 128 < kcp) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) raw[u] = load_raw8<16>(d.W, it.wbase + (int64_t)min(kcur + 128 + rs * 8 + u, kc - 1) * d.ldw).v;
      }
      const V8 af = *reinterpret_cast<const V8*>(&a_s[cv * ka_ld + kcur + rs * 8]);   // row m = lane % 16
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        u32x4 b;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          b[q] = __builtin_amdgcn_perm(cur[2 * q + 1][e >> 1], cur[2 * q][e >> 1], (e & 1) ? 0x07060302u : 0x05040100u);
        acc[e] = TypeTraits<T>::mfma16(af, __builtin_bit_cast(V8, b), acc[e]);
      }
    }
    TR(trb + 2);
    // add the four waves, four fragments at a time; lane l of fragment e holds rows m = 4 (l / 16) + i, column n0 + 8 (l % 16) + e
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<f32x4*>(&red[((wave * 4 + e) * 64 + lane) * 4]) = acc[h * 4 + e];
      __syncthreads();
      {
        const int e = tid >> 6, l = tid & 63;
        f32x4 v = *reinterpret_cast<const f32x4*>(&red[((0 * 4 + e) * 64 + l) * 4]);
        v += *reinterpret_cast<const f32x4*>(&red[((1 * 4 + e) * 64 + l) * 4]);
        v += *reinterpret_cast<const f32x4*>(&red[((2 * 4 + e) * 64 + l) * 4]);
        v += *reinterpret_cast<const f32x4*>(&red[((3 * 4 + e) * 64 + l) * 4]);
        const int gn = n0 + (l & 15) * 8 + h * 4 + e;
        if (gn < d.N) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int m = (l >> 4) * 4 + i;
            if (m < M) {
              if (d.ksplit == 1) emit<T>(d, M, bt, m, gn, v[i], zcur);
              else st_dev(&d.part[(((int64_t)it.ks * d.batch + bt) * M + m) * d.N + gn], v[i]);
            }
          }
        }
      }
    }
    TR(trb + 3);
    kn_splitk_finish<T>(d, M, bt, it.nc, n0, NC, red, zcur, trb);
  }
}

// ---- NK phase (MFMA) ------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ typename TypeTraits<T>::vec8 codes_to_vec8(uint32_t lo, uint32_t hi) {
  typename TypeTraits<T>::vec8 v;
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (T)(float)(int8_t)((lo >> (8 * e)) & 0xFF);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[4 + e] = (T)(float)(int8_t)((hi >> (8 * e)) & 0xFF);
  return v;
}
template <typename T>
__device__ __forceinline__ typename TypeTraits<T>::vec8 nibbles_to_vec8(uint32_t w) {
  typename TypeTraits<T>::vec8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (T)(float)(((int32_t)(w << (28 - 4 * e))) >> 28);
  return v;
}

// Work item of the NK phase: 16 weight rows per wave.  Either the 4 waves take 4 consecutive
// row groups (64 rows per item) or, when that would leave too few items, they split K four ways
// over one row group (16 rows per item) and add their tiles through LDS.
struct NkItem {
  int bt, n, kbeg, kend;
  bool row_ok;
  int64_t row_off;
};
template <int KSTEP>
__device__ __forceinline__ NkItem nk_item(const PhaseDesc& d, int item, int wave, int nl, int Kp) {
  NkItem it;
  const int rows_per_item = d.nk_split_k ? 16 : 64;
  const int rgroups = (d.N + rows_per_item - 1) / rows_per_item;
  const int rg = item % rgroups;
  it.bt = item / rgroups;
  it.n = rg * rows_per_item + (d.nk_split_k ? 0 : wave * 16) + nl;
  it.row_ok = it.n < d.N;
  it.row_off = (int64_t)it.bt * d.w_bs + (int64_t)(it.row_ok ? it.n : 0) * d.ldw;   // clamped: always a valid row
  if (d.nk_split_k) {
    const int steps = Kp / KSTEP, per = (steps + 3) / 4;
    it.kbeg = min(steps, wave * per) * KSTEP;
    it.kend = min(steps, (wave + 1) * per) * KSTEP;
  } else {
    it.kbeg = 0; it.kend = Kp;
  }
  return it;
}

template <int WB>
__device__ __forceinline__ u32x4 nk_load16(const void* W, int64_t row_off, int k) {
  const uint8_t* base = reinterpret_cast<const uint8_t*>(W);
  int64_t byte = (WB == 16) ? (row_off + k) * 2 : (WB == 8 ? (row_off + k) : ((row_off + k) >> 1));
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + byte));
}

template <typename T, int WB, bool VEC>
__device__ __forceinline__ void phase_nk(const PhaseDesc& d, int M, float* smem, float* zcur) {
  using V8 = typename TypeTraits<T>::vec8;
  constexpr int KSTEP = (WB == 16) ? 32 : (WB == 8 ? 64 : 128);   // k per 16-byte lane load x 4 lane groups
  constexpr int LANE_K = KSTEP / 4;                                  // k covered by one lane's 16 bytes
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Kp = (d.K + KSTEP - 1) / KSTEP * KSTEP;
  const int ld = Kp + 8;
  T* a_s = reinterpret_cast<T*>(smem);              // [16][Kp + 8]
  float* tile_red = reinterpret_cast<float*>(a_s + 16 * ld);   // [4 waves][64 lanes][4] (split-K mode)
  const int rows_per_item = d.nk_split_k ? 16 : 64;
  const int total = d.batch * ((d.N + rows_per_item - 1) / rows_per_item);
  const int nl = lane & 15, kg = lane >> 4;
  const int Kfull = d.K / KSTEP * KSTEP;
  int staged_bt = -1;
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const NkItem it = nk_item<KSTEP>(d, item, wave, nl, Kp);
    const int kend_full = min(it.kend, Kfull);
    u32x4 raw[UNR];
    int kk = it.kbeg;
    bool have_raw = false;
    if (VEC && kk + UNR * KSTEP <= kend_full) {       // weights do not depend on the activations: start them first
#pragma unroll
      for (int u = 0; u < UNR; ++u) raw[u] = nk_load16<WB>(d.W, it.row_off, kk + u * KSTEP + kg * LANE_K);
      have_raw = true;
    }
    if (it.bt != staged_bt) {
      __syncthreads();
      for (int idx = tid; idx < 16 * Kp; idx += 256) {
        int m = idx / Kp, k = idx - m * Kp;
        float v = (m < M && k < d.K) ? act_load<T>(d, M, it.bt, m, k, zcur) : 0.0f;
        a_s[m * ld + k] = TypeTraits<T>::from_f32(v);
      }
      __syncthreads();
      staged_bt = it.bt;
    }
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const T* arow = a_s + nl * ld;
    auto consume = [&](const u32x4& c, int k) {      // k = element offset of this lane's 16 bytes
      if (WB == 16) {
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k), __builtin_bit_cast(V8, c), acc);
      } else if (WB == 8) {
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k), codes_to_vec8<T>(c[0], c[1]), acc);
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k + 8), codes_to_vec8<T>(c[2], c[3]), acc);
      } else {
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2)
          acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k + 8 * s2), nibbles_to_vec8<T>(c[s2]), acc);
      }
    };
    if (VEC) {
      while (have_raw) {
        const int kcur = kk;
        kk += UNR * KSTEP;
        const bool more = kk + UNR * KSTEP <= kend_full;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const u32x4 c = raw[u];
          if (more) raw[u] = nk_load16<WB>(d.W, it.row_off, kk + u * KSTEP + kg * LANE_K);   // refill the slot at once
          consume(c, kcur + u * KSTEP + kg * LANE_K);
        }
        have_raw = more;
      }
      for (; kk < it.kend; kk += KSTEP) {            // leftover steps; the last one may be partial
        const int k = kk + kg * LANE_K;
        u32x4 c = {0u, 0u, 0u, 0u};
        if (k + LANE_K <= d.K) c = nk_load16<WB>(d.W, it.row_off, k);
        consume(c, k);
      }
    } else {
      // element-wise path for rows that are not 16-byte friendly (f16/bf16 weights only)
      const T* wrow = reinterpret_cast<const T*>(d.W) + it.row_off;
      for (; kk < it.kend; kk += 32) {
        int k = kk + kg * 8;
        V8 bw;
#pragma unroll
        for (int e = 0; e < 8; ++e) bw[e] = (k + e < d.K) ? wrow[k + e] : (T)0.0f;
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k), bw, acc);
      }
    }
    if (d.nk_split_k) {                              // add the four K-quarters
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 4; ++e) tile_red[(wave * 64 + lane) * 4 + e] = acc[e];
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[e] = tile_red[lane * 4 + e] + tile_red[(64 + lane) * 4 + e] + tile_red[(128 + lane) * 4 + e] + tile_red[(192 + lane) * 4 + e];
      }
    }
    if (it.row_ok && (!d.nk_split_k || wave == 0)) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int m = kg * 4 + e;
        if (m < M) emit<T>(d, M, it.bt, m, it.n, acc[e]);
      }
    }
  }
}

// ---- NK phase, small M: lanes along k, fully coalesced rows, wave reduction ---------------------------
// A wave owns 16 weight rows and walks them four at a time; one load instruction reads 1 KB of
// one row (lane l holds k = 8 l .. 8 l + 7 of each 512-element chunk).  The activation slices a
// lane needs are the same for every row, so they live in registers.
constexpr int dot_kch(int MT) { return MT == 1 ? 4 : 2; }   // 512-element chunks of K kept in registers per lane
__device__ __forceinline__ bool nk_use_dot(const PhaseDesc& d, int MT) {
  return MT <= 4 && d.wbits == 16 && d.vec_ok && (d.K % 8 == 0) && d.K <= 512 * dot_kch(MT) && !d.nk_split_k;
}

template <typename T, int MT>
__device__ __forceinline__ void phase_nk_dot(const PhaseDesc& d, int M, float* smem, float* zcur) {
  float* a_s = smem;                               // [MT][K] fp32
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rgroups = (d.N + 63) / 64;
  const int total = d.batch * rgroups;
  constexpr int DOT_KCH = dot_kch(MT);
  const int kch = (d.K + 511) / 512;               // 512-element chunks per row (<= DOT_KCH)
  int staged_bt = -1;
  float a[DOT_KCH][MT][8];
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const int rg = item % rgroups, bt = item / rgroups;
    const int row0 = rg * 64 + wave * 16;
    const int64_t wb = (int64_t)bt * d.w_bs;
    auto load_group = [&](int g, u32x4 (&raw)[UNR]) {   // rows row0 + 4g .. +3, chunks 0..kch-1 (two passes if kch > 2)
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int r4 = u / 2, c = u % 2;
        const int n = min(row0 + 4 * g + r4, d.N - 1), k = min(c * 512 + lane * 8, d.K - 8);
        raw[u] = nk_load16<16>(d.W, wb + (int64_t)n * d.ldw, k);
      }
    };
    u32x4 raw[UNR];
    load_group(0, raw);
    if (bt != staged_bt) {
      __syncthreads();
      for (int idx = tid; idx < MT * d.K; idx += 256) {
        int m = idx / d.K, k = idx - m * d.K;
        a_s[idx] = (m < M) ? act_load<T>(d, M, bt, m, k, zcur) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int c = 0; c < DOT_KCH; ++c)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int k = c * 512 + lane * 8 + e;
            a[c][m][e] = (c < kch && k < d.K) ? a_s[m * d.K + k] : 0.0f;
          }
      staged_bt = bt;
    }
    for (int g = 0; g < 4; ++g) {
      float acc[4][MT];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[r4][m] = 0.0f;
      // chunks 0 and 1 come from the pipelined registers
      u32x4 cur[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) cur[u] = raw[u];
      if (g < 3) load_group(g + 1, raw);            // next four rows in flight while these are reduced
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int r4 = u / 2, c = u % 2;
        if (c < kch) {
          float w[8];
          raw_to_f32<T>(Raw8<16>{cur[u]}, w);
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[r4][m] = fmaf(a[c][m][e], w[e], acc[r4][m]);
        }
      }
      if (kch > 2) {                                // rare: rank above 1024, chunks 2 and 3 loaded in place
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
          for (int c = 2; c < DOT_KCH; ++c) {
            if (c < kch) {
              const int n = min(row0 + 4 * g + r4, d.N - 1), k = min(c * 512 + lane * 8, d.K - 8);
              float w[8];
              raw_to_f32<T>(Raw8<16>{nk_load16<16>(d.W, wb + (int64_t)n * d.ldw, k)}, w);
#pragma unroll
              for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[r4][m] = fmaf(a[c][m][e], w[e], acc[r4][m]);
            }
          }
      }
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[r4][m] = wave_sum(acc[r4][m]);
      // lane r4 writes row r4
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int n = row0 + 4 * g + r4;
        if (lane == r4 && n < d.N) {
#pragma unroll
          for (int m = 0; m < MT; ++m)
            if (m < M) emit<T>(d, M, bt, m, n, acc[r4][m]);
        }
      }
    }
  }
}

// ---- MIX phase ----------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void phase_mix(const PhaseDesc& d, int M) {
  const T* S = reinterpret_cast<const T*>(d.S);
  float* Z = reinterpret_cast<float*>(d.o);
  if ((d.R & 3) == 0 && d.b <= 16) {
    // Four adjacent lanes share one output (i, m, four consecutive r) and take four j each, so a
    // thread issues four 16-byte device-scope loads in one round; the lanes are then added in a
    // fixed order with two shuffles.
    const int rq = d.R >> 2;
    const int64_t total = (int64_t)d.b * M * rq * 4;
    const int64_t span = ((int64_t)gridDim.x * 256);
    for (int64_t base = (int64_t)blockIdx.x * 256; base < total; base += span) {   // whole workgroups stay in step for the shuffles
      const int64_t idx = base + threadIdx.x;
      const bool live = idx < total;
      const int jq = (int)(idx & 3);
      const int64_t oi = live ? (idx >> 2) : 0;
      const int r = (int)(oi % rq) * 4;
      const int64_t t = oi / rq;
      const int m = (int)(t % M), i = (int)(t / M);
      f32x4 yv[4];
      typename TypeTraits<T>::vec4 sv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jq * 4 + u;
        const bool ok = live && j < d.b;
        yv[u] = ld_dev4(d.Y, ok ? (uint32_t)((((int64_t)j * M + m) * d.R + r) * 4) : 0u);
        if (d.s_sr == 1) {
          sv[u] = *reinterpret_cast<const typename TypeTraits<T>::vec4*>(&S[(int64_t)i * d.s_si + (int64_t)(ok ? j : 0) * d.s_sj + r]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) sv[u][e] = S[(int64_t)i * d.s_si + (int64_t)(ok ? j : 0) * d.s_sj + (int64_t)(r + e) * d.s_sr];
        }
      }
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jq * 4 + u;
        if (live && j < d.b) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float sx = TypeTraits<T>::to_f32(sv[u][e]);
            if (d.v_scales) sx *= (float)d.v_scales[(int64_t)j * d.R + r + e];
            acc[e] = fmaf(sx, yv[u][e], acc[e]);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] += __shfl_xor(acc[e], 1, 64);
        acc[e] += __shfl_xor(acc[e], 2, 64);
      }
      if (live && jq == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) st_dev(&Z[((int64_t)i * M + m) * d.R + r + e], acc[e]);
      }
    }
    return;
  }
  const int64_t total = (int64_t)d.b * M * d.R;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    int r = (int)(idx % d.R);
    int64_t t = idx / d.R;
    int m = (int)(t % M), i = (int)(t / M);
    float acc = 0.0f;
    for (int j = 0; j < d.b; ++j) {
      float sx = TypeTraits<T>::to_f32(S[(int64_t)i * d.s_si + (int64_t)j * d.s_sj + (int64_t)r * d.s_sr]);
      if (d.v_scales) sx *= (float)d.v_scales[(int64_t)j * d.R + r];
      acc = fmaf(sx, ld_dev(&d.Y[((int64_t)j * M + m) * d.R + r]), acc);
    }
    st_dev(&Z[((int64_t)i * M + m) * d.R + r], acc);
  }
}

template <typename T, int MT, int WB, bool VEC>
__device__ __forceinline__ void run_phase(const PhaseDesc& d, int M, float* smem, int trb, float* zcur) {
  if (d.kind == PH_KN) {
    if (WB == 16 && VEC && d.kn_mfma) phase_kn_mfma<T>(d, M, smem, trb, zcur);
    else phase_kn<T, MT, WB, VEC>(d, M, smem, trb, zcur);
  }
  else if (d.kind == PH_NK) {
    if (MT <= 4 && WB == 16 && VEC && nk_use_dot(d, MT)) phase_nk_dot<T, (MT <= 4 ? MT : 1)>(d, M, smem, zcur);
    else phase_nk<T, WB, VEC>(d, M, smem, zcur);
  } else if (d.kind == PH_MIX) phase_mix<T>(d, M);
}

// One kernel per (element type, M tile, weight width, 16-byte-friendly rows): every phase of a call
// shares the weight width, and the element-wise row path is only there for odd or tiny shapes.
template <typename T, int MT, int WB, bool VEC>
__global__ __launch_bounds__(256, 2) void stream_kernel(StreamParams p) {
  extern __shared__ float smem[];
  TR(0);
  unsigned parity = 0;
  float* zcur = nullptr;
  if (p.zatom) {
    parity = __hip_atomic_load(&p.ctrl[Z_PARITY], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 1u;
    zcur = p.zbuf[parity];
    if (p.first) {                                 // zero the other buffer for the next call (nobody reads it in this one)
      const unsigned dirty = __hip_atomic_load(&p.ctrl[Z_DIRTY + (parity ^ 1u)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      float* zoth = p.zbuf[parity ^ 1u];
      for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < dirty; i += gridDim.x * 256) st_dev(&zoth[i], 0.0f);
    }
  }
  for (int ph = 0; ph < p.nph; ++ph) {
    if (ph > 0 && p.use_barrier) { TR(6); grid_barrier(p.ctrl, (unsigned)ph, p.spin_limit); TR(7); }
    run_phase<T, MT, WB, VEC>(p.ph[ph], p.M, smem, ph == 0 ? 0 : 8, zcur);
  }
  TR(15);
  if ((p.use_barrier && p.nph > 1) || (p.zatom && p.finish)) call_finish(p, parity);
}

// ---- host side --------------------------------------------------------------------------------
namespace {

constexpr size_t CTRL_BYTES = 16384;          // barrier shards, finished counters, error word
constexpr int MAX_COUNTERS = 8192;

struct WsLayout {
  unsigned* ctrl; unsigned* counters; float* zb0; float* zb1; void* d2; void* plain; float* buf0; float* buf1; float* part;
};
constexpr size_t ZCAP_FLOATS = 256 * 1024;    // capacity of each fixed-place Z accumulation buffer (1 MiB)

int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
}
// Workgroups kept resident per CU.
int wgs_per_cu() { return 2; }
// Largest M for which the BLAST mix is recomputed inside the last phase instead of run as its own phase.
int mix_inline_max_m() { return 0; }
// Largest M for which BLAST stage 1 adds its S-weighted result straight into Z with float atomics
// (one grid barrier instead of two, no separate mix phase; the summation order over j is then not fixed).
// Off by default: measured slower on MI355X, device-scope float atomics being the bottleneck.
int zatom_max_m() { return 0; }

int nk_kstep(int wbits) { return wbits == 16 ? 32 : (wbits == 8 ? 64 : 128); }

size_t lds_bytes_for(const StreamParams& p) {
  size_t need = 0;
  for (int i = 0; i < p.nph; ++i) {
    const PhaseDesc& d = p.ph[i];
    size_t b = 0;
    if (d.kind == PH_KN && d.kn_mfma) {
      const size_t kcp = (size_t)(d.kc + 127) / 128 * 128;
      b = 16 * (kcp + 8) * 2;                                   // activations as [16][kcp + 8] two-byte values
      if (b < 4 * 4 * 64 * 4 * sizeof(float)) b = 4 * 4 * 64 * 4 * sizeof(float);   // the reduction reuses the same area
    } else if (d.kind == PH_KN) b = (size_t)(AS_FLOATS + 4 * RED_MG * NC_MAX) * sizeof(float);
    else if (d.kind == PH_NK) {
      int ks = nk_kstep(d.wbits);
      int Kp = (d.K + ks - 1) / ks * ks;
      b = (size_t)16 * (Kp + 8) * 2 + 4 * 64 * 4 * sizeof(float);
      size_t dot = (size_t)4 * d.K * sizeof(float);   // small-M path stages fp32 activations
      if (dot > b) b = dot;
    }
    if (b > need) need = b;
  }
  return need;
}

int mt_for(int M) { return M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16))); }

// Choose the KN tiling: lanes per row, k-chunk and split count, aiming at `target` work items.
// Smallest M served by the matrix-core KN variant.
int kn_mfma_min_m() { return 5; }

bool plan_kn(PhaseDesc& d, int MT, int target, int M = 0) {
  const int vecs = (d.N + 7) / 8;
  if (M >= kn_mfma_min_m() && d.wbits == 16 && d.vec_ok && d.K >= 8) {
    d.kn_mfma = 1; d.lpr_log2 = 4;
    d.nchunks = (vecs + 15) / 16;
    if ((int64_t)d.batch * d.nchunks > MAX_COUNTERS / 2) { set_error("stream: too many column chunks"); return false; }
    int split = (int)(target / ((int64_t)d.batch * d.nchunks));
    if (split < 1) split = 1;
    if (split > KSPLIT_MAX) split = KSPLIT_MAX;
    int kc = ((d.K + split - 1) / split + 127) / 128 * 128;
    if (kc > KNM_KC_MAX) kc = KNM_KC_MAX;
    if (kc > d.K) kc = d.K;
    d.kc = kc; d.ksplit = (d.K + kc - 1) / kc;
    if (d.ksplit > KSPLIT_MAX) { set_error("stream: K=%d too deep", d.K); return false; }
    return true;
  }
  const int kc_max = AS_FLOATS / MT;
  int lg_full = 2;
  while ((1 << lg_full) < vecs && lg_full < 6) ++lg_full;   // lanes per row: next pow2 >= N/8 within [4, 64]
  if ((int64_t)d.batch * ((vecs + 3) / 4) > MAX_COUNTERS / 2) { set_error("stream: too many column chunks"); return false; }
  // Option 1: each workgroup owns all of K for a narrower column chunk (row segments of at least
  // 128 bytes).  No partial sums cross workgroups, which takes three memory round trips off the
  // end of the phase.  Taken when it still yields enough workgroups to keep HBM busy.
  const bool allow_nosplit = false;
  if (allow_nosplit && d.K <= kc_max) {
    for (int lg = lg_full; lg >= 3; --lg) {
      const int lpr = 1 << lg;
      const int nch = (vecs + lpr - 1) / lpr;
      if ((int64_t)d.batch * nch * 2 >= target) {
        d.lpr_log2 = lg; d.nchunks = nch; d.kc = d.K; d.ksplit = 1;
        return true;
      }
    }
  }
  // Option 2: widest column chunks, K split across workgroups (partials in slots).
  d.lpr_log2 = lg_full;
  const int lpr = 1 << lg_full, rpp = 256 >> lg_full;
  d.nchunks = (vecs + lpr - 1) / lpr;
  const int64_t base_items = (int64_t)d.batch * d.nchunks;
  int split = (int)(target / base_items);        // never more items than resident workgroups: one round, no straggler pass
  if (split < 1) split = 1;
  if (split > KSPLIT_MAX) split = KSPLIT_MAX;
  int kc = (d.K + split - 1) / split;
  const int batch_rows = UNR * rpp;            // rows one full batch of loads covers
  kc = (kc + batch_rows - 1) / batch_rows * batch_rows;
  if (kc > kc_max) kc = kc_max / batch_rows * batch_rows;
  if (kc < batch_rows) kc = batch_rows < kc_max ? batch_rows : kc_max;
  if (kc > d.K) kc = d.K;
  d.kc = kc;
  d.ksplit = (d.K + kc - 1) / kc;
  if (d.ksplit > KSPLIT_MAX) { set_error("stream: K=%d too deep for M tile %d", d.K, MT); return false; }
  return true;
}

void plan_nk(PhaseDesc& d, int target) {
  d.nk_split_k = ((int64_t)d.batch * ((d.N + 63) / 64) * 2 <= target) ? 1 : 0;
}

template <typename T, int WB, bool VEC>
void* kernel_ptr_mt(int MT) {
  switch (MT) {
    case 1: return (void*)stream_kernel<T, 1, WB, VEC>;
    case 2: return (void*)stream_kernel<T, 2, WB, VEC>;
    case 4: return (void*)stream_kernel<T, 4, WB, VEC>;
    case 8: return (void*)stream_kernel<T, 8, WB, VEC>;
    default: return (void*)stream_kernel<T, 16, WB, VEC>;
  }
}
template <typename T>
void* kernel_ptr(int MT, int wbits, bool vec) {
  if (wbits == 8) return kernel_ptr_mt<T, 8, true>(MT);
  if (wbits == 4) return kernel_ptr_mt<T, 4, true>(MT);
  return vec ? kernel_ptr_mt<T, 16, true>(MT) : kernel_ptr_mt<T, 16, false>(MT);
}

int64_t items_of(const PhaseDesc& d, int M) {
  if (d.kind == PH_KN) return (int64_t)d.batch * d.ksplit * d.nchunks;
  if (d.kind == PH_NK) return (int64_t)d.batch * ((d.N + (d.nk_split_k ? 15 : 63)) / (d.nk_split_k ? 16 : 64));
  if (d.kind == PH_MIX) return ((int64_t)d.b * M * d.R + 255) / 256;   // the vector variant needs exactly this many workgroups too (R/4 * 4 lanes)
  return 0;
}

template <typename T>
int launch_t(StreamParams& p, int MT, int split, hipStream_t st) {
  int wbits = 16;
  bool vec = true;
  for (int i = 0; i < p.nph; ++i) {
    if (p.ph[i].kind == PH_KN || p.ph[i].kind == PH_NK) { wbits = p.ph[i].wbits; vec = vec && p.ph[i].vec_ok; }
  }
  void* fn = kernel_ptr<T>(MT, wbits, vec);
  size_t lds = lds_bytes_for(p);
  // The occupancy of (kernel, LDS size) never changes: ask once, so that steady-state calls are
  // launch-only (and legal under stream capture).
  static std::mutex occ_mu;
  static std::map<std::pair<void*, size_t>, int> occ_cache;
  int occ = 0;
  hipError_t e = hipSuccess;
  {
    std::lock_guard<std::mutex> lk(occ_mu);
    auto it = occ_cache.find({fn, lds});
    if (it != occ_cache.end()) occ = it->second;
    else {
      if (lds > 64 * 1024) {
        e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) { set_error("stream: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
      }
      e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, 256, lds);
      if (e != hipSuccess || occ < 1) { set_error("stream: occupancy query failed"); (void)hipGetLastError(); return BLR_ERR_LAUNCH; }
      occ_cache[{fn, lds}] = occ;
    }
  }
  const int cus = device_cus();
  int per_cu = wgs_per_cu() < occ ? wgs_per_cu() : occ;
  const int resident = per_cu * cus;
  if (split || p.nph == 1) {
    int nph = p.nph;
    StreamParams q = p;
    for (int i = 0; i < nph; ++i) {
      q.ph[0] = p.ph[i]; q.nph = 1; q.use_barrier = 0;
      q.first = (i == 0); q.finish = (i == nph - 1);
      int64_t items = items_of(q.ph[0], p.M);
      int grid = (int)(items < resident ? items : resident);
      if (grid < 1) grid = 1;
      void* args[] = {&q};
      e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st);
      if (e != hipSuccess) { set_error("stream: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    }
    return BLR_OK;
  }
  int64_t most = 0;
  for (int i = 0; i < p.nph; ++i) most = items_of(p.ph[i], p.M) > most ? items_of(p.ph[i], p.M) : most;
  int grid = (int)(most < resident ? most : resident);
  if (grid < 1) grid = 1;
  p.use_barrier = 1; p.first = 1; p.finish = 1;
  void* args[] = {&p};
  e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st);
  if (e != hipSuccess) { set_error("stream: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

int launch(StreamParams& p, int dtype, int split, hipStream_t st) {
  int MT = mt_for(p.M);
  p.spin_limit = spin_limit_now();
  if (dtype == BLR_F16) return launch_t<f16>(p, MT, split, st);
  if (dtype == BLR_BF16) return launch_t<bf16>(p, MT, split, st);
  set_error("stream: dtype %d not supported (f16 / bf16 only)", dtype);
  return BLR_ERR_UNSUPPORTED;
}

int target_items() { return wgs_per_cu() * (device_cus() > 0 ? device_cus() : 256); }

// Workspace: [ctrl][counters][Z ping][Z pong][tagged pairs][plain scratch][buf0][buf1][partials]; everything before buf0 sits at
// fixed offsets and must be zero before the first call (the kernels leave it consistent afterwards).
size_t ws_total(size_t buf_elems, size_t part_elems) {
  return CTRL_BYTES + MAX_COUNTERS * sizeof(unsigned) + 2 * ZCAP_FLOATS * 4 + decode2_region_bytes() + decode2_plain_bytes() +
         align_up(buf_elems * 4, 256) * 2 + align_up(part_elems * 4, 256);
}
WsLayout ws_carve(void* ws, size_t buf_elems) {
  WsLayout l;
  char* p = reinterpret_cast<char*>(ws);
  l.ctrl = reinterpret_cast<unsigned*>(p); p += CTRL_BYTES;
  l.counters = reinterpret_cast<unsigned*>(p); p += MAX_COUNTERS * sizeof(unsigned);
  l.zb0 = reinterpret_cast<float*>(p); p += ZCAP_FLOATS * 4;
  l.zb1 = reinterpret_cast<float*>(p); p += ZCAP_FLOATS * 4;
  l.d2 = p; p += decode2_region_bytes();
  l.plain = p; p += decode2_plain_bytes();
  l.buf0 = reinterpret_cast<float*>(p); p += align_up(buf_elems * 4, 256);
  l.buf1 = reinterpret_cast<float*>(p); p += align_up(buf_elems * 4, 256);
  l.part = reinterpret_cast<float*>(p);
  return l;
}

// Upper bound of split-k partial storage for a KN phase of the given shape (any tiling plan_kn may pick).
size_t part_bound(int M, int batch, int K, int N) {
  size_t ksplit = (size_t)(K + 7) / 8;           // a k-chunk is never shorter than 8 rows unless K is
  if (ksplit > (size_t)KSPLIT_MAX) ksplit = KSPLIT_MAX;
  return ksplit * batch * (size_t)M * N;
}

}  // namespace

// Bytes of the fixed-place block at the start of every streaming workspace (control words, counters, Z buffers, tagged pairs);
// what follows it is per-call scratch.
size_t stream_ws_prefix_bytes() { return ws_total(0, 0); }
size_t stream_ws_error_offset() { return (size_t)BAR_ERR * sizeof(unsigned); }

size_t stream_blast_workspace(int M, int in_f, int out_f, int b, int r, int wbits) {
  (void)wbits;
  size_t buf = (size_t)b * M * r;
  size_t p1 = part_bound(M, b, in_f / b, r);
  size_t p2 = part_bound(M, b, r, out_f / b);
  return ws_total(buf, p1 > p2 ? p1 : p2);
}

int stream_blast_launch(const StreamBlastArgs& a, hipStream_t st) {
  const int P = a.in_f / a.b, Q = a.out_f / a.b;
  size_t need = stream_blast_workspace(a.M, a.in_f, a.out_f, a.b, a.r, a.wbits);
  if (!a.ws || a.ws_bytes < need) { set_error("blast stream: workspace %zu < %zu", a.ws_bytes, need); return BLR_ERR_WORKSPACE; }
  WsLayout w = ws_carve(a.ws, (size_t)a.b * a.M * a.r);
  if (decode2_applicable(a) || a.rows_only) {
    int rc = decode2_blast_launch(a, w.d2, w.plain, w.ctrl + D2_EPOCH, w.ctrl + D2_ARRIVE, w.ctrl + BAR_ERR, st);
    if (rc <= 0) return rc;                    // served (or failed); 1 = shape outside its tiling
  }
  if (a.rows_only) return BLR_ERR_UNSUPPORTED;
  const int MT = mt_for(a.M), target = target_items();
  const bool zatom = a.M <= zatom_max_m() && (size_t)a.b * a.M * a.r <= ZCAP_FLOATS;
  const bool inline_mix = !zatom && a.M <= mix_inline_max_m();
  StreamParams p = {};
  p.M = a.M; p.ctrl = w.ctrl; p.nph = (zatom || inline_mix) ? 2 : 3;
  p.zatom = zatom; p.zbuf[0] = w.zb0; p.zbuf[1] = w.zb1; p.zextent = (unsigned)((size_t)a.b * a.M * a.r);

  PhaseDesc mix = {};                          // Z_i = sum_j S_ij * Y_j
  mix.kind = PH_MIX; mix.Y = w.buf0; mix.S = a.S; mix.b = a.b; mix.R = a.r; mix.o = w.buf1; mix.v_scales = (const f16*)a.v_scales;
  if (a.s_layout == BLR_S_JIR) { mix.s_sj = (int64_t)a.b * a.r; mix.s_si = a.r; mix.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { mix.s_sr = (int64_t)a.b * a.b; mix.s_si = a.b; mix.s_sj = 1; }
  else { mix.s_si = (int64_t)a.b * a.r; mix.s_sj = a.r; mix.s_sr = 1; }

  PhaseDesc& y = p.ph[0];                      // Y_j = x_j V_j
  y.kind = PH_KN; y.wbits = a.wbits; y.W = a.V; y.w_bs = (int64_t)P * a.r; y.ldw = a.r;
  y.batch = a.b; y.K = P; y.N = a.r;
  y.amode = A_X; y.a = a.x; y.lda = a.ldx; y.a_bs = P;
  if (zatom) {
    y.emode = E_ZATOM; y.S = mix.S; y.b = mix.b; y.R = mix.R; y.v_scales = mix.v_scales;
    y.s_si = mix.s_si; y.s_sj = mix.s_sj; y.s_sr = mix.s_sr;
  } else {
    y.emode = E_F32; y.o = w.buf0; y.ldo = a.r;
  }
  y.part = w.part; y.counters = w.counters;
  y.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.V, 16) && a.r % 8 == 0);
  if (!plan_kn(y, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;

  if (p.nph == 3) p.ph[1] = mix;

  PhaseDesc& o = p.ph[p.nph - 1];              // out_i = Z_i U_i
  o.wbits = a.wbits; o.W = a.U; o.batch = a.b; o.K = a.r; o.N = Q;
  if (zatom) {
    o.amode = A_Z;
  } else if (inline_mix) {
    o.amode = A_MIX; o.Y = mix.Y; o.S = mix.S; o.b = mix.b; o.R = mix.R; o.v_scales = mix.v_scales;
    o.s_si = mix.s_si; o.s_sj = mix.s_sj; o.s_sr = mix.s_sr;
  } else {
    o.amode = A_F32; o.a = w.buf1;
  }
  o.emode = E_OUT; o.o = a.out; o.ldo = a.ldo; o.o_bs = Q; o.o_ns = 1;
  o.o_scales = (const f16*)a.u_scales;
  o.part = w.part; o.counters = w.counters + MAX_COUNTERS / 2;
  if (a.u_layout == BLR_U_RQ) {
    o.kind = PH_KN; o.w_bs = (int64_t)a.r * Q; o.ldw = Q;
    o.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.U, 16) && Q % 8 == 0);
    if (!plan_kn(o, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
  } else {
    o.kind = PH_NK; o.w_bs = (int64_t)Q * a.r; o.ldw = a.r;
    o.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.U, 16) && a.r % 8 == 0);
    plan_nk(o, target);
  }
  return launch(p, a.dtype, a.split, st);
}

size_t stream_generic_workspace(int op, int M, int in_f, int out_f, int b, int r) {
  if (op == 0) return ws_total(0, part_bound(M, 1, in_f, out_f));
  if (op == 1) {
    size_t p1 = part_bound(M, 1, in_f, r), p2 = part_bound(M, 1, r, out_f);
    return ws_total((size_t)M * r, p1 > p2 ? p1 : p2);
  }
  size_t p1 = part_bound(M, b, in_f / b, r), p2 = part_bound(M, b, r, out_f / b);
  return ws_total((size_t)b * M * r, p1 > p2 ? p1 : p2);
}

int stream_generic_launch(const StreamGenericArgs& a, hipStream_t st) {
  size_t need = stream_generic_workspace(a.op, a.M, a.in_f, a.out_f, a.b, a.r);
  if (!a.ws || a.ws_bytes < need) { set_error("stream: workspace %zu < %zu", a.ws_bytes, need); return BLR_ERR_WORKSPACE; }
  const int MT = mt_for(a.M), target = target_items();
  StreamParams p = {};
  p.M = a.M;
  if (a.op == 0) {                             // dense: out = x W, W (in, out)
    WsLayout w = ws_carve(a.ws, 0);
    if (!a.split) {                            // the slab kernel (the partial-sum area holds up to KSPLIT_MAX slices, or K / 8)
      const int max_slices = (a.in_f + 7) / 8 < KSPLIT_MAX ? (a.in_f + 7) / 8 : KSPLIT_MAX;
      int rc = dense_slab_launch(a.x, a.ldx, a.W1, a.out, a.ldo, a.M, a.in_f, a.out_f, a.dtype, w.part, max_slices, st);
      if (rc != 1) return rc;
    }
    p.ctrl = w.ctrl; p.nph = 1;
    PhaseDesc& d = p.ph[0];
    d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.w_bs = 0; d.ldw = a.out_f; d.batch = 1; d.K = a.in_f; d.N = a.out_f;
    d.amode = A_X; d.a = a.x; d.lda = a.ldx; d.a_bs = 0;
    d.emode = E_OUT; d.o = a.out; d.ldo = a.ldo; d.o_bs = 0; d.o_ns = 1;
    d.part = w.part; d.counters = w.counters;
    d.vec_ok = aligned(a.W1, 16) && a.out_f % 8 == 0;
    if (!plan_kn(d, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
    return launch(p, a.dtype, a.split, st);
  }
  if (a.op == 1) {                             // low rank: z = x A (in, r); out = z B (r, out)
    WsLayout w = ws_carve(a.ws, (size_t)a.M * a.r);
    constexpr int rows_min_m = 2;
    if (!a.split && a.M >= rows_min_m) {
      // From two rows up: the three-launch matrix-core path, low rank being BLAST with the input cut into 16 (or 8, 4, 2) slices of
      // rows of A, one output block and S = 1 (the mix is the sum over the slices).
      int bi = 0;
      for (int c = 16; c >= 2 && !bi; c >>= 1)
        if (a.in_f % c == 0 && (a.in_f / c) % 8 == 0) bi = c;
      if (bi) {
        StreamBlastArgs bl = {};
        bl.x = a.x; bl.ldx = a.ldx; bl.U = a.W2; bl.V = a.W1; bl.S = nullptr; bl.out = a.out; bl.ldo = a.ldo;
        bl.M = a.M; bl.in_f = a.in_f; bl.out_f = a.out_f; bl.b = bi; bl.bo = 1; bl.r = a.r;
        bl.dtype = a.dtype; bl.u_layout = BLR_U_RQ; bl.s_layout = BLR_S_IJR; bl.wbits = 16;
        const int rc = decode_rows_launch(bl, w.plain, decode2_plain_bytes(), st);
        if (rc != 1) return rc;
      }
    }
    constexpr int slab_min_m = 5;
    if (!a.split && a.M >= slab_min_m && a.r % 8 == 0 && a.out_f % 8 == 0) {
      // From a handful of rows up, two launches of the slab kernel, each followed by the sum of its k-slices: z = x A goes
      // to the first staging buffer as T, then out = z B.  Four launches, 19-29 us whatever M is; the single launch below
      // hands up to 16 rows of intermediates between workgroups and needs 25-39 us at 5..16 rows (measured on the three
      // Llama-7B shapes: ahead everywhere except 4096 -> 22016 at 5 and 8 rows, where it is 1.5 us behind).  The
      // partial-sum area is sized for either product.
      const int s1 = (a.in_f + 7) / 8 < KSPLIT_MAX ? (a.in_f + 7) / 8 : KSPLIT_MAX;
      const int s2 = (a.r + 7) / 8 < KSPLIT_MAX ? (a.r + 7) / 8 : KSPLIT_MAX;
      int rc = slab_gemm_launch(a.x, a.ldx, 0, a.W1, a.r, 0, w.buf0, a.r, 0, a.M, a.r, a.in_f, 1, a.dtype, w.part, s1, st);
      if (rc == BLR_OK) rc = slab_gemm_launch(w.buf0, a.r, 0, a.W2, a.out_f, 0, a.out, a.ldo, 0, a.M, a.out_f, a.r, 1, a.dtype, w.part, s2, st);
      if (rc != 1) return rc;                   // 1: not for the slab kernel - the paths below compute the whole layer
    }
    if (!a.split) {
      // The two-stage decode kernel sees a low-rank layer as a BLAST layer with the input cut into
      // blocks of rows of A, a single output block and S = 1.
      int bi = 0;
      for (int c = 16; c >= 2 && !bi; c >>= 1)
        if (a.in_f % c == 0 && (a.in_f / c) % 8 == 0) bi = c;
      if (bi) {
        StreamBlastArgs bl = {};
        bl.x = a.x; bl.ldx = a.ldx; bl.U = a.W2; bl.V = a.W1; bl.S = nullptr; bl.out = a.out; bl.ldo = a.ldo;
        bl.M = a.M; bl.in_f = a.in_f; bl.out_f = a.out_f; bl.b = bi; bl.bo = 1; bl.r = a.r;
        bl.dtype = a.dtype; bl.u_layout = BLR_U_RQ; bl.s_layout = BLR_S_IJR; bl.wbits = 16;
        if (decode2_applicable(bl)) {
          int rc = decode2_blast_launch(bl, w.d2, w.plain, w.ctrl + D2_EPOCH, w.ctrl + D2_ARRIVE, w.ctrl + BAR_ERR, st);
          if (rc <= 0) return rc;
        }
      }
    }
    p.ctrl = w.ctrl; p.nph = 2;
    PhaseDesc& d = p.ph[0];
    d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.ldw = a.r; d.batch = 1; d.K = a.in_f; d.N = a.r;
    d.amode = A_X; d.a = a.x; d.lda = a.ldx;
    d.emode = E_F32; d.o = w.buf0; d.ldo = a.r;
    d.part = w.part; d.counters = w.counters;
    d.vec_ok = aligned(a.W1, 16) && a.r % 8 == 0;
    if (!plan_kn(d, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
    PhaseDesc& e = p.ph[1];
    e.kind = PH_KN; e.wbits = 16; e.W = a.W2; e.ldw = a.out_f; e.batch = 1; e.K = a.r; e.N = a.out_f;
    e.amode = A_F32; e.a = w.buf0;
    e.emode = E_OUT; e.o = a.out; e.ldo = a.ldo; e.o_ns = 1;
    e.part = w.part; e.counters = w.counters + MAX_COUNTERS / 2;
    e.vec_ok = aligned(a.W2, 16) && a.out_f % 8 == 0;
    if (!plan_kn(e, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
    return launch(p, a.dtype, a.split, st);
  }
  // Monarch: out1 = scatter(x_k w1_k); out = out1_l w2_l
  const int P = a.in_f / a.b, S = a.out_f / a.b, per = a.r / a.b;
  WsLayout w = ws_carve(a.ws, (size_t)a.b * a.M * a.r);
  if (!a.split && a.w2_layout == BLR_W2_RS && a.b >= 2 && a.r % a.b == 0) {
    // Two-stage decode kernel: a BLAST-shaped call whose mix is the Monarch permutation.
    StreamBlastArgs bl = {};
    bl.x = a.x; bl.ldx = a.ldx; bl.U = a.W2; bl.V = a.W1; bl.S = nullptr; bl.out = a.out; bl.ldo = a.ldo;
    bl.M = a.M; bl.in_f = a.in_f; bl.out_f = a.out_f; bl.b = a.b; bl.bo = a.b; bl.r = a.r;
    bl.dtype = a.dtype; bl.u_layout = BLR_U_RQ; bl.s_layout = BLR_S_IJR; bl.wbits = 16;
    bl.perm_per = per;
    if (a.out_order == BLR_OUT_INTERLEAVED) { bl.out_bs = 1; bl.out_ns = a.b; }
    else { bl.out_bs = S; bl.out_ns = 1; }
    if (decode2_applicable(bl)) {
      int rc = decode2_blast_launch(bl, w.d2, w.plain, w.ctrl + D2_EPOCH, w.ctrl + D2_ARRIVE, w.ctrl + BAR_ERR, st);
      if (rc <= 0) return rc;
    }
  }
  p.ctrl = w.ctrl; p.nph = 2;
  PhaseDesc& d = p.ph[0];
  d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.w_bs = (int64_t)P * a.r; d.ldw = a.r; d.batch = a.b; d.K = P; d.N = a.r;
  d.amode = A_X; d.a = a.x; d.lda = a.ldx; d.a_bs = P;
  d.emode = E_F32; d.o = w.buf0; d.ldo = a.r; d.perm_per = per;
  d.part = w.part; d.counters = w.counters;
  d.vec_ok = aligned(a.W1, 16) && a.r % 8 == 0;
  if (!plan_kn(d, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
  PhaseDesc& e = p.ph[1];
  e.wbits = 16; e.W = a.W2; e.batch = a.b; e.K = a.r; e.N = S;
  e.amode = A_F32; e.a = w.buf0;
  e.emode = E_OUT; e.o = a.out; e.ldo = a.ldo;
  if (a.out_order == BLR_OUT_INTERLEAVED) { e.o_bs = 1; e.o_ns = a.b; }
  else { e.o_bs = S; e.o_ns = 1; }
  e.part = w.part; e.counters = w.counters + MAX_COUNTERS / 2;
  if (a.w2_layout == BLR_W2_RS) {
    e.kind = PH_KN; e.w_bs = (int64_t)a.r * S; e.ldw = S;
    e.vec_ok = aligned(a.W2, 16) && S % 8 == 0;
    if (!plan_kn(e, MT, target, a.M)) return BLR_ERR_UNSUPPORTED;
  } else {
    e.kind = PH_NK; e.w_bs = (int64_t)S * a.r; e.ldw = a.r;
    e.vec_ok = aligned(a.W2, 16) && a.r % 8 == 0;
    plan_nk(e, target);
  }
  return launch(p, a.dtype, a.split, st);
}

// ---- bandwidth probe ------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void probe_kernel(const u32x4* __restrict__ src, size_t nvec, uint32_t* __restrict__ dst) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  size_t stride = (size_t)gridDim.x * 256 * 4;
  size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
  for (; i + 3 * 256 < nvec; i += stride) {
    u32x4 a = __builtin_nontemporal_load(&src[i]);
    u32x4 b = __builtin_nontemporal_load(&src[i + 256]);
    u32x4 c = __builtin_nontemporal_load(&src[i + 512]);
    u32x4 e = __builtin_nontemporal_load(&src[i + 768]);
    acc ^= a ^ b ^ c ^ e;
  }
  uint32_t v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  for (int o = 32; o > 0; o >>= 1) v ^= __shfl_xor(v, o, 64);
  if ((threadIdx.x & 63) == 0) atomicXor(&dst[blockIdx.x], v);
}

// Loads every byte of up to three operands with the streaming pattern and stores zeros over all of y: the memory traffic
// of a layer (activations in, factors in, result out) without its arithmetic.  The stored value depends on the loaded
// data (it is zero unless the checksum hits one particular value), so no load can be dropped.
struct ProbeSrc { const u32x4* p; size_t nvec; };
__global__ __launch_bounds__(256) void load_store_probe_kernel(ProbeSrc s0, ProbeSrc s1, ProbeSrc s2, u32x4* __restrict__ y, size_t yvec,
                                                               uint32_t* __restrict__ dst) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  const ProbeSrc srcs[3] = {s0, s1, s2};
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const u32x4* src = srcs[k].p;
    const size_t nvec = srcs[k].nvec;
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
    for (; i + 3 * 256 < nvec; i += stride) {
      u32x4 a = __builtin_nontemporal_load(&src[i]);
      u32x4 b = __builtin_nontemporal_load(&src[i + 256]);
      u32x4 c = __builtin_nontemporal_load(&src[i + 512]);
      u32x4 e = __builtin_nontemporal_load(&src[i + 768]);
      acc ^= a ^ b ^ c ^ e;
    }
    for (; i < nvec; i += 256) acc ^= __builtin_nontemporal_load(&src[i]);      // the last, short block of four
  }
  uint32_t v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  for (int o = 32; o > 0; o >>= 1) v ^= __shfl_xor(v, o, 64);
  if ((threadIdx.x & 63) == 0) atomicXor(&dst[blockIdx.x], v);
  const uint32_t z = (v == 0x9E3779B9u && acc[0] == 0x85EBCA6Bu) ? 1u : 0u;
  const u32x4 zero = {z, z, z, z};
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < yvec; i += (size_t)gridDim.x * 256) __builtin_nontemporal_store(zero, &y[i]);
}

}  // namespace blr

#ifdef BLR_TRACE
extern "C" int blr_debug_trace(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(blr::g_trace), (size_t)n * 8, 0, hipMemcpyDeviceToHost);
}
#endif

extern "C" int blr_probe_dst_words(void) { return 2 * blr::device_cus() > 0 ? 2 * blr::device_cus() : 512; }

extern "C" int blr_load_store_probe(const void* x, size_t x_bytes, const void* w1, size_t w1_bytes, const void* w2, size_t w2_bytes,
                                    void* y, size_t y_bytes, void* dst, void* stream) {
  if (!x || !w1 || !y || !dst || (w2_bytes && !w2)) { blr::set_error("load_store_probe: null pointer"); return BLR_ERR_BAD_ARG; }
  if ((x_bytes | w1_bytes | w2_bytes | y_bytes) % 16 || !blr::aligned(x, 16) || !blr::aligned(w1, 16) || !blr::aligned(y, 16) ||
      (w2 && !blr::aligned(w2, 16))) {
    blr::set_error("load_store_probe: operands must be whole 16-byte pieces at 16-byte addresses");
    return BLR_ERR_BAD_ARG;
  }
  const int grid = blr_probe_dst_words();
  const blr::ProbeSrc s0 = {(const blr::u32x4*)x, x_bytes / 16}, s1 = {(const blr::u32x4*)w1, w1_bytes / 16},
                      s2 = {(const blr::u32x4*)w2, w2 ? w2_bytes / 16 : 0};
  hipLaunchKernelGGL(blr::load_store_probe_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, s0, s1, s2,
                     (blr::u32x4*)y, y_bytes / 16, (uint32_t*)dst);
  BLR_CHECK_LAUNCH("load_store_probe");
  return BLR_OK;
}

extern "C" int blr_stream_probe(const void* src, size_t bytes, void* dst, void* stream) {
  if (!src || !dst || bytes < 16) { blr::set_error("probe: bad argument"); return BLR_ERR_BAD_ARG; }
  int grid = blr_probe_dst_words();
  hipLaunchKernelGGL(blr::probe_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const blr::u32x4*)src, bytes / 16, (uint32_t*)dst);
  BLR_CHECK_LAUNCH("probe");
  return BLR_OK;
}

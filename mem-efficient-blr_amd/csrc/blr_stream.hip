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
//   MIX : BLAST rank-space mix  Z_i = sum_j S_ij * Y_j  (tiny; its own phase so it runs once).
// Intermediates (Y, Z, low-rank z, Monarch out1) are fp32 in the caller's workspace and stay
// in L2 / Infinity Cache.
#include "blr_common.h"

namespace blr {

enum { PH_NONE = 0, PH_KN = 1, PH_NK = 2, PH_MIX = 3 };
enum { A_X = 0, A_F32 = 1 };
enum { E_F32 = 0, E_OUT = 1 };

constexpr int KC_MAX = 256;     // rows of a KN slab held in LDS as fp32 activations
constexpr int NC_MAX = 512;     // widest KN column chunk (64 lanes x 8)
constexpr int RED_MG = 4;       // activation rows reduced across waves per pass
constexpr unsigned SPIN_LIMIT = 400000u;

struct PhaseDesc {
  int kind, wbits;
  const void* W; int64_t w_bs, ldw;         // element (code) units
  int batch, K, N;
  int lpr_log2, kc, ksplit, nchunks;        // KN tiling
  int amode; const void* a; int64_t lda, a_bs;
  int emode; void* o; int64_t ldo, o_bs, o_ns;
  int perm_per;                             // > 0: Monarch scatter on E_F32
  const f16* o_scales;                      // per (bt, n) output scale or null
  float* part; unsigned* counters;
  const float* Y; const void* S; int64_t s_si, s_sj, s_sr; int b, R; const f16* v_scales;   // MIX
  int vec_ok;
};

struct StreamParams {
  PhaseDesc ph[3];
  int nph, M, use_barrier;
  unsigned* ctrl;                           // [0] barrier arrivals, [1] finished workgroups, [2] error flag
};

// ---- grid barrier ---------------------------------------------------------------------------
// All workgroups of the launch are resident (the host sizes the grid from the occupancy query),
// so every arrival is eventually seen.  The wait is bounded: on expiry the error word is set and
// the workgroup carries on, so the grid always drains.
__device__ __forceinline__ void grid_barrier(unsigned* ctrl, unsigned target) {
  // Every wave publishes its own stores device-wide (they may sit in another XCD's L2 otherwise)
  // before the workgroup reports in, and drops stale cache lines after the wait.
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    __hip_atomic_fetch_add(&ctrl[0], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    unsigned spins = 0;
    while (__hip_atomic_load(&ctrl[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(1);
      if (++spins > SPIN_LIMIT) {
        __hip_atomic_store(&ctrl[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
  }
  __syncthreads();
  __threadfence();
}

// ---- weight fetch: 8 consecutive elements as float --------------------------------------------
template <typename T>
__device__ __forceinline__ void fetch8(const PhaseDesc& d, int64_t eoff, int nvalid, float (&w)[8]) {
  if (d.wbits == 16) {
    const T* p = reinterpret_cast<const T*>(d.W) + eoff;
    if (d.vec_ok) {
      typename TypeTraits<T>::vec8 v = ldg16<typename TypeTraits<T>::vec8>(p);
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = TypeTraits<T>::to_f32(v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = (e < nvalid) ? TypeTraits<T>::to_f32(p[e]) : 0.0f;
    }
  } else if (d.wbits == 8) {
    const int8_t* p = reinterpret_cast<const int8_t*>(d.W) + eoff;
    u32x2 v = *reinterpret_cast<const u32x2*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = (float)(int8_t)((v[e >> 2] >> ((e & 3) * 8)) & 0xFF);
  } else {
    const uint8_t* p = reinterpret_cast<const uint8_t*>(d.W) + (eoff >> 1);
    uint32_t v = *reinterpret_cast<const uint32_t*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = (float)(((int32_t)(v << (28 - 4 * e))) >> 28);
  }
}

template <typename T>
__device__ __forceinline__ void emit(const PhaseDesc& d, int M, int bt, int m, int n, float v) {
  if (d.o_scales) v *= (float)d.o_scales[(int64_t)bt * d.N + n];
  if (d.emode == E_OUT) {
    reinterpret_cast<T*>(d.o)[(int64_t)m * d.ldo + (int64_t)bt * d.o_bs + (int64_t)n * d.o_ns] = TypeTraits<T>::from_f32(v);
  } else {
    float* o = reinterpret_cast<float*>(d.o);
    if (d.perm_per > 0) {
      int dst = n / d.perm_per, j = n - dst * d.perm_per;
      o[((int64_t)dst * M + m) * d.ldo + (int64_t)bt * d.perm_per + j] = v;
    } else {
      o[((int64_t)bt * M + m) * d.ldo + n] = v;
    }
  }
}

template <typename T>
__device__ __forceinline__ float act_load(const PhaseDesc& d, int M, int bt, int m, int k) {
  if (d.amode == A_X) return TypeTraits<T>::to_f32(reinterpret_cast<const T*>(d.a)[(int64_t)m * d.lda + (int64_t)bt * d.a_bs + k]);
  return reinterpret_cast<const float*>(d.a)[((int64_t)bt * M + m) * d.K + k];
}

// ---- KN phase -----------------------------------------------------------------------------------
template <typename T, int MT>
__device__ void phase_kn(const PhaseDesc& d, int M, float* smem) {
  float* a_s = smem;                               // [MT][KC_MAX]
  float* red = smem + MT * KC_MAX;                 // [4 waves][RED_MG][NC_MAX]
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lpr = 1 << d.lpr_log2, rpp = 256 >> d.lpr_log2;
  const int cv = tid & (lpr - 1), rs = tid >> d.lpr_log2;
  const int NC = lpr * 8;
  const int total = d.batch * d.ksplit * d.nchunks;
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const int nc = item % d.nchunks;
    const int t2 = item / d.nchunks;
    const int ks = t2 % d.ksplit, bt = t2 / d.ksplit;
    const int k0 = ks * d.kc, kc = min(d.kc, d.K - k0);
    const int n0 = nc * NC;
    __syncthreads();
    for (int idx = tid; idx < MT * kc; idx += 256) {
      int m = idx / kc, kk = idx - m * kc;
      a_s[m * KC_MAX + kk] = (m < M) ? act_load<T>(d, M, bt, m, k0 + kk) : 0.0f;
    }
    __syncthreads();

    float acc[MT][8];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[m][e] = 0.0f;
    const int n = n0 + cv * 8;
    if (n < d.N) {
      const int nvalid = min(8, d.N - n);
      const int64_t wbase = (int64_t)bt * d.w_bs + (int64_t)k0 * d.ldw + n;
      for (int kk = rs; kk < kc; kk += 4 * rpp) {
        float w[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          int k = kk + u * rpp;
          if (k < kc) fetch8<T>(d, wbase + (int64_t)k * d.ldw, nvalid, w[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          int k = kk + u * rpp;
          if (k < kc) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              float a = a_s[m * KC_MAX + k];
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[m][e] = fmaf(a, w[u][e], acc[m][e]);
            }
          }
        }
      }
    }
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
          if (d.ksplit == 1) emit<T>(d, M, bt, m, gn, v);
          else d.part[(((int64_t)ks * d.batch + bt) * M + m) * d.N + gn] = v;
        }
      }
    }
    if (d.ksplit > 1) {
      __threadfence();
      __syncthreads();
      if (tid == 0) {
        unsigned old = __hip_atomic_fetch_add(&d.counters[bt * d.nchunks + nc], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (unsigned)(d.ksplit - 1));
      }
      __syncthreads();
      if (s_last) {
        __threadfence();
        for (int idx = tid; idx < NC * M; idx += 256) {
          int m = idx / NC, col = idx - m * NC;
          int gn = n0 + col;
          if (gn >= d.N) continue;
          float v = 0.0f;
          for (int s = 0; s < d.ksplit; ++s)
            v += __builtin_nontemporal_load(&d.part[(((int64_t)s * d.batch + bt) * M + m) * d.N + gn]);
          emit<T>(d, M, bt, m, gn, v);
        }
        if (tid == 0) __hip_atomic_store(&d.counters[bt * d.nchunks + nc], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
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

template <typename T>
__device__ void phase_nk(const PhaseDesc& d, int M, float* smem) {
  using V8 = typename TypeTraits<T>::vec8;
  T* a_s = reinterpret_cast<T*>(smem);              // [16][Kp + 8]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kstep = (d.wbits == 16) ? 32 : (d.wbits == 8 ? 64 : 128);   // k consumed per 16-byte lane load x 4 lane groups
  const int Kp = (d.K + kstep - 1) / kstep * kstep;
  const int ld = Kp + 8;
  const int rgroups = (d.N + 63) / 64;
  const int total = d.batch * rgroups;
  const int nl = lane & 15, kg = lane >> 4;
  int staged_bt = -1;
  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    const int rg = item % rgroups, bt = item / rgroups;
    if (bt != staged_bt) {
      __syncthreads();
      for (int idx = tid; idx < 16 * Kp; idx += 256) {
        int m = idx / Kp, k = idx - m * Kp;
        float v = (m < M && k < d.K) ? act_load<T>(d, M, bt, m, k) : 0.0f;
        a_s[m * ld + k] = TypeTraits<T>::from_f32(v);
      }
      __syncthreads();
      staged_bt = bt;
    }
    const int n = rg * 64 + wave * 16 + nl;
    const bool row_ok = n < d.N;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const T* arow = a_s + nl * ld;
    if (d.wbits == 16) {
      const T* wrow = reinterpret_cast<const T*>(d.W) + (int64_t)bt * d.w_bs + (int64_t)(row_ok ? n : 0) * d.ldw;
#pragma unroll 8
      for (int kk = 0; kk < Kp; kk += 32) {
        int k = kk + kg * 8;
        V8 bw;
        if (d.vec_ok) {
          if (row_ok && k < d.K) bw = ldg16<V8>(wrow + k);
          else {
#pragma unroll
            for (int e = 0; e < 8; ++e) bw[e] = (T)0.0f;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) bw[e] = (row_ok && k + e < d.K) ? wrow[k + e] : (T)0.0f;
        }
        V8 aw = *reinterpret_cast<const V8*>(arow + k);
        acc = TypeTraits<T>::mfma16(aw, bw, acc);
      }
    } else if (d.wbits == 8) {
      const int8_t* wrow = reinterpret_cast<const int8_t*>(d.W) + (int64_t)bt * d.w_bs + (int64_t)(row_ok ? n : 0) * d.ldw;
#pragma unroll 4
      for (int kk = 0; kk < Kp; kk += 64) {
        int k = kk + kg * 16;                       // this lane's 16 codes
        u32x4 c = {0u, 0u, 0u, 0u};
        if (row_ok && k < d.K) c = *reinterpret_cast<const u32x4*>(wrow + k);
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k), codes_to_vec8<T>(c[0], c[1]), acc);
        acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k + 8), codes_to_vec8<T>(c[2], c[3]), acc);
      }
    } else {
      const uint8_t* wrow = reinterpret_cast<const uint8_t*>(d.W) + (((int64_t)bt * d.w_bs + (int64_t)(row_ok ? n : 0) * d.ldw) >> 1);
#pragma unroll 2
      for (int kk = 0; kk < Kp; kk += 128) {
        int k = kk + kg * 32;                       // this lane's 32 codes
        u32x4 c = {0u, 0u, 0u, 0u};
        if (row_ok && k < d.K) c = *reinterpret_cast<const u32x4*>(wrow + (k >> 1));
#pragma unroll
        for (int s = 0; s < 4; ++s)
          acc = TypeTraits<T>::mfma16(*reinterpret_cast<const V8*>(arow + k + 8 * s), nibbles_to_vec8<T>(c[s]), acc);
      }
    }
    if (row_ok) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int m = kg * 4 + e;
        if (m < M) emit<T>(d, M, bt, m, n, acc[e]);
      }
    }
  }
}

// ---- MIX phase ----------------------------------------------------------------------------------
template <typename T>
__device__ void phase_mix(const PhaseDesc& d, int M) {
  const int64_t total = (int64_t)d.b * M * d.R;
  const T* S = reinterpret_cast<const T*>(d.S);
  float* Z = reinterpret_cast<float*>(d.o);
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    int r = (int)(idx % d.R);
    int64_t t = idx / d.R;
    int m = (int)(t % M), i = (int)(t / M);
    float acc = 0.0f;
    for (int j = 0; j < d.b; ++j) {
      float s = TypeTraits<T>::to_f32(S[(int64_t)i * d.s_si + (int64_t)j * d.s_sj + (int64_t)r * d.s_sr]);
      if (d.v_scales) s *= (float)d.v_scales[(int64_t)j * d.R + r];
      acc = fmaf(s, d.Y[((int64_t)j * M + m) * d.R + r], acc);
    }
    Z[((int64_t)i * M + m) * d.R + r] = acc;
  }
}

template <typename T, int MT>
__global__ __launch_bounds__(256) void stream_kernel(StreamParams p) {
  extern __shared__ float smem[];
  for (int ph = 0; ph < p.nph; ++ph) {
    if (ph > 0 && p.use_barrier) grid_barrier(p.ctrl, (unsigned)ph * gridDim.x);
    const PhaseDesc& d = p.ph[ph];
    if (d.kind == PH_KN) phase_kn<T, MT>(d, p.M, smem);
    else if (d.kind == PH_NK) phase_nk<T>(d, p.M, smem);
    else if (d.kind == PH_MIX) phase_mix<T>(d, p.M);
  }
  if (p.use_barrier && p.nph > 1) {
    // last workgroup out re-arms the barrier words for the next call
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned old = __hip_atomic_fetch_add(&p.ctrl[1], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (old == gridDim.x - 1) {
        __hip_atomic_store(&p.ctrl[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&p.ctrl[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// ---- host side --------------------------------------------------------------------------------
namespace {

constexpr size_t CTRL_BYTES = 256;
constexpr int MAX_COUNTERS = 8192;

struct WsLayout {
  unsigned* ctrl; unsigned* counters; float* buf0; float* buf1; float* part;
  size_t buf_elems, part_elems;
};

size_t lds_bytes_for(const StreamParams& p, int MT) {
  size_t need = 0;
  for (int i = 0; i < p.nph; ++i) {
    const PhaseDesc& d = p.ph[i];
    size_t b = 0;
    if (d.kind == PH_KN) b = (size_t)(MT * KC_MAX + 4 * RED_MG * NC_MAX) * sizeof(float);
    else if (d.kind == PH_NK) {
      int kstep = (d.wbits == 16) ? 32 : (d.wbits == 8 ? 64 : 128);
      int Kp = (d.K + kstep - 1) / kstep * kstep;
      b = (size_t)16 * (Kp + 8) * 2;
    }
    if (b > need) need = b;
  }
  return need;
}

int mt_for(int M) { return M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16))); }

// Choose the KN tiling: lanes per row, k-chunk and split count.
void plan_kn(PhaseDesc& d, int M, int grid_hint) {
  int vecs = (d.N + 7) / 8;
  int lg = 0;
  while ((1 << lg) < vecs && lg < 6) ++lg;     // lanes per row: next pow2 >= N/8, capped at 64
  if (lg < 2) lg = 2;
  d.lpr_log2 = lg;
  int lpr = 1 << lg, rpp = 256 >> lg;
  d.nchunks = (vecs + lpr - 1) / lpr;
  // aim for ~2 slabs per resident workgroup, each at least 4 passes of the row slots deep
  int64_t base_items = (int64_t)d.batch * d.nchunks;
  int want_split = (int)((2 * (int64_t)grid_hint + base_items - 1) / base_items);
  if (want_split < 1) want_split = 1;
  int kc = (d.K + want_split - 1) / want_split;
  int min_kc = 4 * rpp;
  if (kc < min_kc) kc = min_kc;
  kc = (kc + rpp - 1) / rpp * rpp;
  if (kc > KC_MAX) kc = KC_MAX;
  if (kc > d.K) kc = d.K;
  d.kc = kc;
  d.ksplit = (d.K + kc - 1) / kc;
  (void)M;
}

template <typename T>
void* kernel_ptr(int MT) {
  switch (MT) {
    case 1: return (void*)stream_kernel<T, 1>;
    case 2: return (void*)stream_kernel<T, 2>;
    case 4: return (void*)stream_kernel<T, 4>;
    case 8: return (void*)stream_kernel<T, 8>;
    default: return (void*)stream_kernel<T, 16>;
  }
}

template <typename T>
int launch_t(StreamParams& p, int MT, int split, hipStream_t st) {
  void* fn = kernel_ptr<T>(MT);
  size_t lds = lds_bytes_for(p, MT);
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { set_error("stream: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  }
  int occ = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, 256, lds);
  if (e != hipSuccess || occ < 1) { set_error("stream: occupancy query failed"); (void)hipGetLastError(); return BLR_ERR_LAUNCH; }
  int cus = device_cus();
  int resident = occ * cus;
  if (occ > 2) resident = 2 * cus;              // two workgroups per CU already saturate the load queues
  auto items_of = [&](const PhaseDesc& d) -> int64_t {
    if (d.kind == PH_KN) return (int64_t)d.batch * d.ksplit * d.nchunks;
    if (d.kind == PH_NK) return (int64_t)d.batch * ((d.N + 63) / 64);
    if (d.kind == PH_MIX) return ((int64_t)d.b * p.M * d.R + 255) / 256;
    return 0;
  };
  if (split || p.nph == 1) {
    int nph = p.nph;
    StreamParams q = p;
    for (int i = 0; i < nph; ++i) {
      q.ph[0] = p.ph[i]; q.nph = 1; q.use_barrier = 0;
      int64_t items = items_of(q.ph[0]);
      int grid = (int)(items < resident ? items : resident);
      if (grid < 1) grid = 1;
      void* args[] = {&q};
      e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st);
      if (e != hipSuccess) { set_error("stream: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    }
    return BLR_OK;
  }
  int64_t most = 0;
  for (int i = 0; i < p.nph; ++i) most = items_of(p.ph[i]) > most ? items_of(p.ph[i]) : most;
  int grid = (int)(most < resident ? most : resident);
  if (grid < 1) grid = 1;
  p.use_barrier = 1;
  void* args[] = {&p};
  e = hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st);
  if (e != hipSuccess) { set_error("stream: launch failed: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  return BLR_OK;
}

int launch(StreamParams& p, int dtype, int split, hipStream_t st) {
  int MT = mt_for(p.M);
  if (dtype == BLR_F16) return launch_t<f16>(p, MT, split, st);
  if (dtype == BLR_BF16) return launch_t<bf16>(p, MT, split, st);
  set_error("stream: dtype %d not supported (f16 / bf16 only)", dtype);
  return BLR_ERR_UNSUPPORTED;
}

// Workspace: [ctrl 256 B][counters][buf0][buf1][partials]
size_t ws_total(size_t buf_elems, size_t part_elems) {
  return CTRL_BYTES + MAX_COUNTERS * sizeof(unsigned) + align_up(buf_elems * 4, 256) * 2 + align_up(part_elems * 4, 256);
}
WsLayout ws_carve(void* ws, size_t buf_elems, size_t part_elems) {
  WsLayout l;
  char* p = reinterpret_cast<char*>(ws);
  l.ctrl = reinterpret_cast<unsigned*>(p); p += CTRL_BYTES;
  l.counters = reinterpret_cast<unsigned*>(p); p += MAX_COUNTERS * sizeof(unsigned);
  l.buf0 = reinterpret_cast<float*>(p); p += align_up(buf_elems * 4, 256);
  l.buf1 = reinterpret_cast<float*>(p); p += align_up(buf_elems * 4, 256);
  l.part = reinterpret_cast<float*>(p);
  l.buf_elems = buf_elems; l.part_elems = part_elems;
  return l;
}

// Upper bound of split-K partial storage for a KN phase of the given shape (any tiling plan_kn may pick).
size_t part_bound(int M, int batch, int K, int N) {
  // ksplit <= ceil(K / min_kc) with min_kc >= 16 (4 passes of >= 4 row slots)
  size_t ksplit = (size_t)(K + 15) / 16;
  if (ksplit > 64) ksplit = 64;
  return ksplit * batch * (size_t)M * N;
}

// Keep the split count within the bound the workspace was sized for.
bool cap_split(PhaseDesc& d) {
  while (d.ksplit > 64 && d.kc < KC_MAX) {
    d.kc = d.kc * 2 > KC_MAX ? KC_MAX : d.kc * 2;
    d.ksplit = (d.K + d.kc - 1) / d.kc;
  }
  return d.ksplit <= 64;
}

}  // namespace

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
  size_t p1 = part_bound(a.M, a.b, P, a.r), p2 = part_bound(a.M, a.b, a.r, Q);
  WsLayout w = ws_carve(a.ws, (size_t)a.b * a.M * a.r, p1 > p2 ? p1 : p2);
  const int cus = device_cus();
  StreamParams p = {};
  p.M = a.M; p.ctrl = w.ctrl; p.nph = 3;

  PhaseDesc& y = p.ph[0];                      // Y_j = x_j V_j
  y.kind = PH_KN; y.wbits = a.wbits; y.W = a.V; y.w_bs = (int64_t)P * a.r; y.ldw = a.r;
  y.batch = a.b; y.K = P; y.N = a.r;
  y.amode = A_X; y.a = a.x; y.lda = a.ldx; y.a_bs = P;
  y.emode = E_F32; y.o = w.buf0; y.ldo = a.r;
  y.part = w.part; y.counters = w.counters;
  y.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.V, 16) && a.r % 8 == 0);
  plan_kn(y, a.M, 2 * cus); if (!cap_split(y)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }

  PhaseDesc& z = p.ph[1];                      // Z_i = sum_j S_ij * Y_j
  z.kind = PH_MIX; z.Y = w.buf0; z.S = a.S; z.b = a.b; z.R = a.r; z.o = w.buf1; z.v_scales = (const f16*)a.v_scales;
  if (a.s_layout == BLR_S_JIR) { z.s_sj = (int64_t)a.b * a.r; z.s_si = a.r; z.s_sr = 1; }
  else if (a.s_layout == BLR_S_RIJ) { z.s_sr = (int64_t)a.b * a.b; z.s_si = a.b; z.s_sj = 1; }
  else { z.s_si = (int64_t)a.b * a.r; z.s_sj = a.r; z.s_sr = 1; }

  PhaseDesc& o = p.ph[2];                      // out_i = Z_i U_i
  o.wbits = a.wbits; o.W = a.U; o.batch = a.b; o.K = a.r; o.N = Q;
  o.amode = A_F32; o.a = w.buf1;
  o.emode = E_OUT; o.o = a.out; o.ldo = a.ldo; o.o_bs = Q; o.o_ns = 1;
  o.o_scales = (const f16*)a.u_scales;
  o.part = w.part; o.counters = w.counters + MAX_COUNTERS / 2;
  if (a.u_layout == BLR_U_RQ) {
    o.kind = PH_KN; o.w_bs = (int64_t)a.r * Q; o.ldw = Q;
    o.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.U, 16) && Q % 8 == 0);
    plan_kn(o, a.M, 2 * cus); if (!cap_split(o)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
  } else {
    o.kind = PH_NK; o.w_bs = (int64_t)Q * a.r; o.ldw = a.r;
    o.vec_ok = (a.wbits != 16) ? 1 : (aligned(a.U, 16) && a.r % 8 == 0);
  }
  if ((int64_t)y.batch * y.nchunks > MAX_COUNTERS / 2 || (o.kind == PH_KN && (int64_t)o.batch * o.nchunks > MAX_COUNTERS / 2)) {
    set_error("blast stream: too many column chunks for the counter table");
    return BLR_ERR_UNSUPPORTED;
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
  const int cus = device_cus();
  StreamParams p = {};
  p.M = a.M;
  if (a.op == 0) {                             // dense: out = x W, W (in, out)
    WsLayout w = ws_carve(a.ws, 0, part_bound(a.M, 1, a.in_f, a.out_f));
    p.ctrl = w.ctrl; p.nph = 1;
    PhaseDesc& d = p.ph[0];
    d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.w_bs = 0; d.ldw = a.out_f; d.batch = 1; d.K = a.in_f; d.N = a.out_f;
    d.amode = A_X; d.a = a.x; d.lda = a.ldx; d.a_bs = 0;
    d.emode = E_OUT; d.o = a.out; d.ldo = a.ldo; d.o_bs = 0; d.o_ns = 1;
    d.part = w.part; d.counters = w.counters;
    d.vec_ok = aligned(a.W1, 16) && a.out_f % 8 == 0;
    plan_kn(d, a.M, 2 * cus); if (!cap_split(d)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
    if (d.nchunks > MAX_COUNTERS) { set_error("dense stream: out_f too wide"); return BLR_ERR_UNSUPPORTED; }
    return launch(p, a.dtype, a.split, st);
  }
  if (a.op == 1) {                             // low rank: z = x A (in, r); out = z B (r, out)
    size_t p1 = part_bound(a.M, 1, a.in_f, a.r), p2 = part_bound(a.M, 1, a.r, a.out_f);
    WsLayout w = ws_carve(a.ws, (size_t)a.M * a.r, p1 > p2 ? p1 : p2);
    p.ctrl = w.ctrl; p.nph = 2;
    PhaseDesc& d = p.ph[0];
    d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.ldw = a.r; d.batch = 1; d.K = a.in_f; d.N = a.r;
    d.amode = A_X; d.a = a.x; d.lda = a.ldx;
    d.emode = E_F32; d.o = w.buf0; d.ldo = a.r;
    d.part = w.part; d.counters = w.counters;
    d.vec_ok = aligned(a.W1, 16) && a.r % 8 == 0;
    plan_kn(d, a.M, 2 * cus); if (!cap_split(d)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
    PhaseDesc& e = p.ph[1];
    e.kind = PH_KN; e.wbits = 16; e.W = a.W2; e.ldw = a.out_f; e.batch = 1; e.K = a.r; e.N = a.out_f;
    e.amode = A_F32; e.a = w.buf0;
    e.emode = E_OUT; e.o = a.out; e.ldo = a.ldo; e.o_ns = 1;
    e.part = w.part; e.counters = w.counters + MAX_COUNTERS / 2;
    e.vec_ok = aligned(a.W2, 16) && a.out_f % 8 == 0;
    plan_kn(e, a.M, 2 * cus); if (!cap_split(e)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
    if (d.nchunks > MAX_COUNTERS / 2 || e.nchunks > MAX_COUNTERS / 2) { set_error("low rank stream: too wide"); return BLR_ERR_UNSUPPORTED; }
    return launch(p, a.dtype, a.split, st);
  }
  // Monarch: out1 = scatter(x_k w1_k); out = out1_l w2_l
  const int P = a.in_f / a.b, S = a.out_f / a.b, per = a.r / a.b;
  size_t p1 = part_bound(a.M, a.b, P, a.r), p2 = part_bound(a.M, a.b, a.r, S);
  WsLayout w = ws_carve(a.ws, (size_t)a.b * a.M * a.r, p1 > p2 ? p1 : p2);
  p.ctrl = w.ctrl; p.nph = 2;
  PhaseDesc& d = p.ph[0];
  d.kind = PH_KN; d.wbits = 16; d.W = a.W1; d.w_bs = (int64_t)P * a.r; d.ldw = a.r; d.batch = a.b; d.K = P; d.N = a.r;
  d.amode = A_X; d.a = a.x; d.lda = a.ldx; d.a_bs = P;
  d.emode = E_F32; d.o = w.buf0; d.ldo = a.r; d.perm_per = per;
  d.part = w.part; d.counters = w.counters;
  d.vec_ok = aligned(a.W1, 16) && a.r % 8 == 0;
  plan_kn(d, a.M, 2 * cus); if (!cap_split(d)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
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
    plan_kn(e, a.M, 2 * cus); if (!cap_split(e)) { set_error("stream: K too deep"); return BLR_ERR_UNSUPPORTED; }
  } else {
    e.kind = PH_NK; e.w_bs = (int64_t)S * a.r; e.ldw = a.r;
    e.vec_ok = aligned(a.W2, 16) && a.r % 8 == 0;
  }
  if ((int64_t)d.batch * d.nchunks > MAX_COUNTERS / 2 || (e.kind == PH_KN && (int64_t)e.batch * e.nchunks > MAX_COUNTERS / 2)) {
    set_error("monarch stream: too many column chunks"); return BLR_ERR_UNSUPPORTED;
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

}  // namespace blr

extern "C" int blr_probe_dst_words(void) { return 2 * blr::device_cus() > 0 ? 2 * blr::device_cus() : 512; }

extern "C" int blr_stream_probe(const void* src, size_t bytes, void* dst, void* stream) {
  if (!src || !dst || bytes < 16) { blr::set_error("probe: bad argument"); return BLR_ERR_BAD_ARG; }
  int grid = blr_probe_dst_words();
  hipLaunchKernelGGL(blr::probe_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const blr::u32x4*)src, bytes / 16, (uint32_t*)dst);
  BLR_CHECK_LAUNCH("probe");
  return BLR_OK;
}

// Shared device/host helpers for libblr (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/blr.h"

namespace blr {

typedef _Float16 f16;
typedef __bf16 bf16;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

template <typename T> struct TypeTraits;
template <> struct TypeTraits<f16> {
  using vec8 = f16x8;
  using vec4 = f16x4;
  static __device__ __forceinline__ float to_f32(f16 v) { return (float)v; }
  static __device__ __forceinline__ f16 from_f32(float v) { return (f16)v; }
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct TypeTraits<bf16> {
  using vec8 = bf16x8;
  using vec4 = bf16x4;
  static __device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }
  static __device__ __forceinline__ bf16 from_f32(float v) { return (bf16)v; }
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct TypeTraits<float> {
  static __device__ __forceinline__ float to_f32(float v) { return v; }
  static __device__ __forceinline__ float from_f32(float v) { return v; }
};

// Round to nearest even, then clamp to the int8 range (reference blast_sym_quant_kernels.py:105-108: nearbyint, clamp).
__device__ __forceinline__ float sat8_rne(float v) { return fminf(fmaxf(rintf(v), -128.0f), 127.0f); }

// Activation of the fused output stage (blr_act): GELU with the tanh approximation (what the reference's DiT uses,
// DiT/models.py:111: approx_gelu = nn.GELU(approximate="tanh")) or SiLU (Llama's gate).
__device__ __forceinline__ float apply_act(float v, int act) {
  // 0.5 v (1 + tanh u) = v / (1 + exp(-2u)), u = sqrt(2/pi) (v + 0.044715 v^3): one exponential and one reciprocal
  if (act == BLR_ACT_GELU_TANH) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-1.5957691216057308f * (v + 0.044715f * v * v * v)));
  if (act == BLR_ACT_SILU) return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
  return v;
}

// 16-byte global load / store of 8 two-byte elements (pointer must be 16-byte aligned).
template <typename V> __device__ __forceinline__ V ldg16(const void* p) {
  return *reinterpret_cast<const V*>(p);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- host side ------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int device_cus();
// Polls after which a bounded wait inside a kernel gives up and sets the error word of its workspace (blr_set_spin_limit).
unsigned spin_limit_now();
// The fused output stage armed by the *_fwd_ep entry point of the running call, if any (bias of dtype or null, blr_act); a kernel
// that applies it itself says so with epilogue_taken(), otherwise the entry point finishes with an elementwise launch.
bool epilogue_pending(const void** bias, int* act);   // (false when a gate or a residual is armed: only the tiled path fuses those)
void epilogue_taken();
// Every run-time switch of the library (blr_set_option): each starts from the environment variable of its name, read once, and
// is range-checked where it is set.  The first six pick the GEMM variant, the rest switch a kernel family off (0) so that the
// call falls through to the next one that serves it - for A/B measurements and as a way out should a kernel misbehave.
enum { OPT_GEMM_RING = 0, OPT_GEMM_RING_TILE, OPT_GEMM_RING_PER_CU, OPT_GEMM_RING_WAVES, OPT_GEMM_RING_BK, OPT_GEMM_SPLITK,
       OPT_DECODE2, OPT_DECODE3, OPT_DECODE_PAIR, OPT_DECODE_ROWS, OPT_DENSE_SLAB, OPT_DENSE_ROWS, OPT_BLAST_MIXU, OPT_BLAST_ONE, OPT_BLAST_YMIXW, OPT_COUNT };
int option_value(int id, int dflt);             // the option's value, or dflt when it is unset
// true when p is aligned to `bytes`.
static inline bool aligned(const void* p, size_t bytes) { return (reinterpret_cast<uintptr_t>(p) % bytes) == 0; }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define BLR_CHECK_LAUNCH(what)                                              \
  do {                                                                      \
    hipError_t e__ = hipGetLastError();                                     \
    if (e__ != hipSuccess) {                                                \
      blr::set_error("%s: launch failed: %s", what, hipGetErrorString(e__)); \
      return BLR_ERR_LAUNCH;                                                \
    }                                                                       \
  } while (0)

// ---- a small job that rides along with a GEMM launch -------------------------------------------------------------
// What blast_mixu_kernel wants re-laid before it runs (U (16, Q, R) -> Ut (i, rank / 8, q, 8); S(i, j, r) with any strides ->
// Sp (r / 2, j / 4, i, r % 2, 4)) depends on the weights only, and the GEMM x V that precedes it in the same call touches neither:
// extra workgroups of that GEMM's launch do it, which saves a launch of its own (4.7 us for 1.6 MB: start-up and one trip
// to memory).  items: 16-byte pieces of Ut, then 8-byte pieces of Sp; 0 = no job.
struct SidePrep {
  const void* U; const void* S; void* Ut; void* Sp;
  int Q, R;
  int u_rq;          // U comes as (16, R, Q) instead of (16, Q, R)
  int64_t s_si, s_sj, s_sr;
  int64_t items;
};
template <typename T>
__device__ __forceinline__ void side_prep_item(const SidePrep& s, int64_t idx) {
  const T* U = reinterpret_cast<const T*>(s.U); const T* S = reinterpret_cast<const T*>(s.S);
  T* Ut = reinterpret_cast<T*>(s.Ut); T* Sp = reinterpret_cast<T*>(s.Sp);
  const int R8 = s.R / 8, Q = s.Q;
  const int64_t nu = (int64_t)16 * R8 * Q;
  if (idx < nu && s.u_rq) {                         // U (i, r, q): neighbouring threads take neighbouring columns q, eight ranks each
    const int q = (int)(idx % Q), o = (int)((idx / Q) % R8), i = (int)(idx / ((int64_t)Q * R8));
    typename TypeTraits<T>::vec8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = U[((int64_t)i * s.R + 8 * o + e) * Q + q];
    *reinterpret_cast<typename TypeTraits<T>::vec8*>(Ut + idx * 8) = v;
  } else if (idx < nu) {                            // U (i, q, r): neighbouring threads read neighbouring pieces of a row of U
    const int o = (int)(idx % R8), q = (int)((idx / R8) % Q), i = (int)(idx / ((int64_t)Q * R8));
    *reinterpret_cast<u32x4*>(Ut + (((int64_t)i * R8 + o) * Q + q) * 8) = *reinterpret_cast<const u32x4*>(U + idx * 8);
  } else if (idx - nu < (int64_t)s.R * 64) {
    const int64_t k = idx - nu;
    const int l = (int)(k & 63), r = (int)(k >> 6), n = l & 15, g = l >> 4;
#pragma unroll
    for (int t = 0; t < 4; ++t) Sp[(((int64_t)(r >> 1) * 64 + l) * 2 + (r & 1)) * 4 + t] = S[(int64_t)n * s.s_si + (int64_t)(4 * g + t) * s.s_sj + (int64_t)r * s.s_sr];
  }
}

// ---- tiled GEMM (blr_gemm.hip) ----------------------------------------------------------
enum { EPI_PLAIN = 0, EPI_MONARCH_SCATTER = 1 };
struct GemmArgs {
  const void* A; int64_t lda; int64_t sA;   // A[bt*sA + m*lda + k]
  const void* B; int64_t ldb; int64_t sB;   // b_kn: B[bt*sB + k*ldb + n]   else: B[bt*sB + n*ldb + k]
  void* C; int64_t ldc; int64_t sC; int64_t cn;   // C[bt*sC + m*ldc + n*cn]
  int M, N, K, batch;
  int b_kn;
  int epi;          // EPI_*
  int per;          // EPI_MONARCH_SCATTER: column c of batch kk -> C[(c/per)*sL + m*ldc + kk*per + c%per]
  int64_t sL;
  int sat8;         // 1: the fp32 result is rounded to nearest even and clamped to [-128, 127] before it is stored
  const void* bias; // optional: values of dtype added to the rounded result, indexed by the element's offset inside its row of C
  int act;          // blr_act applied after the bias
  const void* gate; int gate_rows; int64_t ld_gate;   // optional: after the activation, the value is multiplied by gate[(m / gate_rows) * ld_gate + offset in row]
  const void* resid; int64_t ld_resid;   // optional: and resid[m * ld_resid + offset in row] is added (DiT: x + g * h, reference DiT/models.py:120-121)
  // pair: every work item computes two tiles one after the other - the same rows and columns of two problems whose operands lie
  // pair_dA / pair_dB elements apart (BLAST: output blocks i and i + b/2; dense and low rank: the columns n and n + N of a factor
  // with 2 N columns) - and writes ONE tile of C: silu(first + bias[..]) * (second + bias[.. + pair_dbias]), the gated unit of
  // Llama's MLP over a fused gate|up projection.  N, batch and C describe one half.  Ring kernels with an output stage only.
  int pair; int64_t pair_dA, pair_dB, pair_dbias;
  void* splitk_ws;  // optional scratch for splitting the reduction (gemm_splitk_bytes says how much); null: never split
  size_t splitk_bytes;
  int kc;           // set by gemm_launch for the split kernels: k values per slice
  SidePrep side;    // optional job for extra workgroups of the launch (items > 0); *side_taken is set to 1 by a launch that carries it
  int* side_taken;  // (host pointer; the kernels that cannot carry the job leave it alone and the caller launches it itself)
};
// dtype: blr_dtype.  Returns blr_status.
int gemm_launch(const GemmArgs& a, int dtype, hipStream_t st);
// Scratch a plain single GEMM M x N x K of dtype wants in GemmArgs::splitk_ws so that a problem with few output tiles and
// a long reduction can be cut along K to fill the chip (fp32 partial results, summed in a fixed order).  0: no split.
size_t gemm_splitk_bytes(int M, int N, int K, int dtype);

// ---- BLAST rank-space mix, tiled path (blr_gemm.hip) ------------------------------------
// Z[i, m, r] = sum_j S(i, j, r) * Y[j, m, r];  Y, Z (b, M, R) contiguous of dtype.
// sat8: accumulate in fp32, then round to nearest even and clamp to [-128, 127] before the store.
int blast_mix_launch(const void* Y, const void* S, void* Z, int M, int b, int R,
                     int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype, hipStream_t st, int sat8 = 0);

// ---- BLAST above 16 rows: Z = mix(S, x V) in one launch, Y never written (blr_prefill.hip) ---------------
// Z (b, M, R) of dtype.  Returns BLR_OK, a negative blr_status, or 1 when the shape is not for the kernel.
// scratch: b * b * R elements for S in (r, i, j) order (not touched when S already has that layout).
int blast_ymix_launch(const void* x, int64_t ldx, const void* V, const void* S, void* Z, int M, int in_f, int b, int R,
                      int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                      hipStream_t st);
int blast_ymixw_launch(const void* x, int64_t ldx, const void* V, const void* S, void* Z, int M, int in_f, int b, int R,
                      int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                      hipStream_t st);
// Second half for output blocks of at most 80 columns: out_i = mix(S, Y)_i U_i with U (b, Q, R) (u_rq: (b, R, Q)), in one launch and without Z;
// the fused output stage (bias, act, gate, resid) is taken from `ep`.  Same return convention; scratch as above.
int blast_mixu_launch(const void* Y, const void* S, const void* U, void* out, int64_t ldo, const GemmArgs& ep, int M, int b, int R, int Q,
                      int64_t s_si, int64_t s_sj, int64_t s_sr, int s_layout, int dtype, void* scratch, size_t scratch_bytes,
                      hipStream_t st, bool prepared = false, bool u_rq = false);
// Whether blast_mixu_launch takes the shape, and the job that re-lays U and S into `scratch` for it (what a GEMM launch earlier
// in the call may carry; blast_mixu_launch is then told `prepared`).
bool blast_mixu_plan(const void* Y, const void* S, const void* U, const void* out, int64_t ldo, const GemmArgs& ep, int M, int b, int R, int Q,
                     int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype, void* scratch, size_t scratch_bytes, SidePrep* job, bool u_rq = false);

// The whole BLAST call in one launch for 16 input blocks of at most 96 columns and 16 output blocks of at most 80 (U (b, Q, R)):
// neither Y nor Z in memory.  scratch: room for V, U and S re-laid.  Same return convention as the two above.
int blast_one_launch(const void* x, int64_t ldx, const void* U, const void* V, const void* S, void* out, int64_t ldo, const GemmArgs& ep,
                     int M, int in_f, int b, int R, int Q, int64_t s_si, int64_t s_sj, int64_t s_sr, int dtype,
                     void* scratch, size_t scratch_bytes, hipStream_t st, bool u_rq = false);

// ---- streaming (decode) engine (blr_stream.hip) -------------------------------------------
struct StreamBlastArgs {
  const void* x; int64_t ldx;
  const void* U; const void* V; const void* S;
  const void* u_scales; const void* v_scales;   // quantized only (fp16)
  void* out; int64_t ldo;
  int M, in_f, out_f, b, r;
  int bo;                                       // output blocks when they differ from b (0: same); S may then be null (all ones)
  int perm_per;                                 // > 0: Monarch - the mix is the permutation with this period, S is unused
  int64_t out_bs, out_ns;                       // output strides of (block, column); out_ns == 0: blocked (bs = q, ns = 1)
  int dtype, u_layout, s_layout;
  int wbits;                                    // 16 = floating weights, 8 / 4 = codes
  void* ws; size_t ws_bytes;
  int split;                                    // 1: separate launches per phase
  int rows_only;                                // 1: only the three-launch matrix-core path may serve the call (codes whose rows are not whole 16-byte pieces)
};
size_t stream_blast_workspace(int M, int in_f, int out_f, int b, int r, int wbits);
size_t stream_ws_prefix_bytes();                // the fixed-place block at the start of a streaming workspace; per-call scratch follows
size_t stream_ws_error_offset();                // byte offset of the error word inside a streaming workspace
int stream_blast_launch(const StreamBlastArgs& a, hipStream_t st);

struct StreamGenericArgs {                      // dense / low-rank / monarch at M <= 16
  const void* x; int64_t ldx;
  const void* W1; const void* W2;               // dense: W1 only
  void* out; int64_t ldo;
  int M, in_f, out_f, b, r;                     // dense: r = 0; low rank: b = 1
  int dtype;
  int op;                                       // 0 dense, 1 low rank, 2 monarch
  int w2_layout, out_order;                     // monarch
  void* ws; size_t ws_bytes;
  int split;
};
size_t stream_generic_workspace(int op, int M, int in_f, int out_f, int b, int r);
int stream_generic_launch(const StreamGenericArgs& a, hipStream_t st);

}  // namespace blr

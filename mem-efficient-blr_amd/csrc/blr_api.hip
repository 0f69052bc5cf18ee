// extern "C" entry points of libblr: argument validation, algorithm choice, workspace carving.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include "blr_common.h"
#include "blr_decode.h"

namespace blr {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int device_cus() {
  static std::once_flag once;
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return 0; }
  std::call_once(once, [] {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return; }
    for (int d = 0; d < n && d < 64; ++d) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, d) == hipSuccess) cus[d] = v;
    }
  });
  return cus[dev];
}

static int elt_size(int dtype) { return dtype == BLR_F32 ? 4 : 2; }
static bool dtype_ok(int dtype) { return dtype == BLR_F16 || dtype == BLR_BF16 || dtype == BLR_F32; }

// ---- quantizer --------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float ld_f32(const T* p, int64_t i) { return TypeTraits<T>::to_f32(p[i]); }

__device__ __forceinline__ int quant_code(float w, float s, float qmax) {
  float q = rintf(__fdiv_rn(w, s));
  q = fminf(fmaxf(q, -qmax), qmax);
  return (int)q;
}
__device__ __forceinline__ float make_scale(float amax, float qmax, f16* store) {
  f16 s16 = (f16)__fdiv_rn(amax, qmax);
  if ((float)s16 == 0.0f) s16 = (f16)1.0f;
  *store = s16;
  return (float)s16;
}

// inner == 1: one workgroup per channel row, max over the contiguous axis.
template <typename T>
__global__ __launch_bounds__(256) void quant_rows_kernel(const T* __restrict__ w, int64_t reduce, int bits,
                                                         uint8_t* __restrict__ codes, f16* __restrict__ scales) {
  __shared__ float s_max[4];
  __shared__ float s_scale;
  const int64_t row = blockIdx.x;
  const T* wr = w + row * reduce;
  float amax = 0.0f;
  for (int64_t k = threadIdx.x; k < reduce; k += 256) amax = fmaxf(amax, fabsf(ld_f32(wr, k)));
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
  if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  const float qmax = bits == 8 ? 127.0f : 7.0f;
  if (threadIdx.x == 0) {
    float m = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    s_scale = make_scale(m, qmax, &scales[row]);
  }
  __syncthreads();
  const float s = s_scale;
  if (bits == 8) {
    int8_t* c = reinterpret_cast<int8_t*>(codes) + row * reduce;
    for (int64_t k = threadIdx.x; k < reduce; k += 256) c[k] = (int8_t)quant_code(ld_f32(wr, k), s, qmax);
  } else {
    uint8_t* c = codes + row * (reduce / 2);
    for (int64_t k = threadIdx.x; k < reduce / 2; k += 256) {
      int lo = quant_code(ld_f32(wr, 2 * k), s, qmax), hi = quant_code(ld_f32(wr, 2 * k + 1), s, qmax);
      c[k] = (uint8_t)((lo & 0xF) | ((hi & 0xF) << 4));
    }
  }
}

// inner > 1: thread per inner column (or column pair for int4), max over the strided axis.
template <typename T>
__global__ __launch_bounds__(256) void quant_cols_kernel(const T* __restrict__ w, int64_t reduce, int64_t inner, int bits,
                                                         uint8_t* __restrict__ codes, f16* __restrict__ scales) {
  const int64_t o = blockIdx.y;
  const int per = bits == 8 ? 1 : 2;
  const int64_t c0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * per;
  if (c0 >= inner) return;
  const T* wo = w + o * reduce * inner;
  const float qmax = bits == 8 ? 127.0f : 7.0f;
  float amax[2] = {0.0f, 0.0f};
  for (int64_t k = 0; k < reduce; ++k)
    for (int u = 0; u < per; ++u) amax[u] = fmaxf(amax[u], fabsf(ld_f32(wo, k * inner + c0 + u)));
  float s[2];
  for (int u = 0; u < per; ++u) s[u] = make_scale(amax[u], qmax, &scales[o * inner + c0 + u]);
  if (bits == 8) {
    int8_t* c = reinterpret_cast<int8_t*>(codes) + o * reduce * inner;
    for (int64_t k = 0; k < reduce; ++k) c[k * inner + c0] = (int8_t)quant_code(ld_f32(wo, k * inner + c0), s[0], qmax);
  } else {
    uint8_t* c = codes + o * reduce * (inner / 2);
    for (int64_t k = 0; k < reduce; ++k) {
      int lo = quant_code(ld_f32(wo, k * inner + c0), s[0], qmax), hi = quant_code(ld_f32(wo, k * inner + c0 + 1), s[1], qmax);
      c[k * (inner / 2) + c0 / 2] = (uint8_t)((lo & 0xF) | ((hi & 0xF) << 4));
    }
  }
}

// codes (rows, cols) -> T; scale index = (row / rows_per_scale_block) * cols + col when per_col, else row.
// cols % 8 == 0: a thread expands 8 consecutive codes (8 or 4 bytes in, 16 bytes out).
template <typename T>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ codes, const f16* __restrict__ scales,
                                                      T* __restrict__ out, int64_t rows, int64_t cols, int bits,
                                                      int per_col, int64_t rows_per_block) {
  using V8 = typename TypeTraits<T>::vec8;
  const int64_t total = rows * cols / 8;
  for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < total; v += (int64_t)gridDim.x * 256) {
    const int64_t idx = v * 8;
    const int64_t row = idx / cols, col = idx - row * cols;
    int c[8];
    if (bits == 8) {
      const u32x2 w = *reinterpret_cast<const u32x2*>(codes + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) c[e] = (int)(int8_t)((w[e >> 2] >> ((e & 3) * 8)) & 0xFF);
    } else {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(codes + (idx >> 1));
#pragma unroll
      for (int e = 0; e < 8; ++e) c[e] = ((int32_t)(w << (28 - 4 * e))) >> 28;
    }
    V8 o;
    if (per_col) {
      const f16x8 sc = *reinterpret_cast<const f16x8*>(&scales[(row / rows_per_block) * cols + col]);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32((float)c[e] * (float)sc[e]);
    } else {
      const float sc = (float)scales[row];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = TypeTraits<T>::from_f32((float)c[e] * sc);
    }
    *reinterpret_cast<V8*>(&out[idx]) = o;
  }
}

template <typename T>
static int quantize_t(const void* w, int64_t outer, int64_t reduce, int64_t inner, int bits, void* codes, void* scales, hipStream_t st) {
  if (inner == 1) {
    hipLaunchKernelGGL(quant_rows_kernel<T>, dim3((unsigned)outer), dim3(256), 0, st, (const T*)w, reduce, bits, (uint8_t*)codes, (f16*)scales);
  } else {
    int per = bits == 8 ? 1 : 2;
    dim3 grid((unsigned)cdiv(cdiv(inner, per), 256), (unsigned)outer);
    hipLaunchKernelGGL(quant_cols_kernel<T>, grid, dim3(256), 0, st, (const T*)w, reduce, inner, bits, (uint8_t*)codes, (f16*)scales);
  }
  BLR_CHECK_LAUNCH("quantize");
  return BLR_OK;
}

// ---- fused output stage ------------------------------------------------------------------------------
// The *_fwd_ep entry points arm this per-thread record and call the plain entry point; the tiled path attaches it
// to its last GEMM (attach_epilogue), any other path leaves it and the entry point finishes with bias_act_kernel.
struct PendingEpilogue { const void* bias; int act; bool armed; bool used; const void* gate; int gate_rows; int64_t ld_gate; const void* resid; int64_t ld_resid; };
static thread_local PendingEpilogue tl_ep = {nullptr, 0, false, false, nullptr, 0, 0, nullptr, 0};

static bool silu_mul_armed() { return tl_ep.armed && tl_ep.act == BLR_ACT_SILU_MUL; }

bool epilogue_pending(const void** bias, int* act) {
  if (!tl_ep.armed || tl_ep.used || tl_ep.gate || tl_ep.resid || tl_ep.act == BLR_ACT_SILU_MUL) return false;
  *bias = tl_ep.bias; *act = tl_ep.act;
  return true;
}
void epilogue_taken() { tl_ep.used = true; }

static void attach_epilogue_peek(GemmArgs& g) {      // the armed output stage, without claiming it
  if (!tl_ep.armed) return;
  g.bias = tl_ep.bias; g.act = tl_ep.act;
  if (tl_ep.act == BLR_ACT_SILU_MUL) { g.act = BLR_ACT_SILU; g.pair = 1; }   // (the caller sets the distances between the halves)
  g.gate = tl_ep.gate; g.gate_rows = tl_ep.gate_rows; g.ld_gate = tl_ep.ld_gate; g.resid = tl_ep.resid; g.ld_resid = tl_ep.ld_resid;
}
static void attach_epilogue(GemmArgs& g) {
  if (!tl_ep.armed) return;
  attach_epilogue_peek(g);
  tl_ep.used = true;
}

template <typename T>
__global__ __launch_bounds__(256) void bias_act_kernel(T* __restrict__ out, int64_t ldo, const T* __restrict__ bias, int act, int M, int N,
                                                        const T* __restrict__ gate, int gate_rows, int64_t ld_gate, const T* __restrict__ resid, int64_t ld_resid) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * N) return;
  const int m = (int)(idx / N), n = (int)(idx - (int64_t)m * N);
  float v = TypeTraits<T>::to_f32(out[(int64_t)m * ldo + n]);
  if (bias) v += TypeTraits<T>::to_f32(bias[n]);
  v = apply_act(v, act);
  if (gate || resid) {
    v = TypeTraits<T>::to_f32(TypeTraits<T>::from_f32(v));
    if (gate) v *= TypeTraits<T>::to_f32(gate[(int64_t)(m / gate_rows) * ld_gate + n]);
    if (resid) v += TypeTraits<T>::to_f32(resid[(int64_t)m * ld_resid + n]);
  }
  out[(int64_t)m * ldo + n] = TypeTraits<T>::from_f32(v);
}

static int bias_act_launch(void* out, int64_t ldo, const PendingEpilogue& ep, int M, int N, int dtype, hipStream_t st) {
  if (!ep.bias && !ep.act && !ep.gate && !ep.resid) return BLR_OK;
  const unsigned grid = (unsigned)cdiv((int64_t)M * N, 256);
  if (dtype == BLR_F16) hipLaunchKernelGGL(bias_act_kernel<f16>, dim3(grid), dim3(256), 0, st, (f16*)out, ldo, (const f16*)ep.bias, ep.act, M, N, (const f16*)ep.gate, ep.gate_rows, ep.ld_gate, (const f16*)ep.resid, ep.ld_resid);
  else if (dtype == BLR_BF16) hipLaunchKernelGGL(bias_act_kernel<bf16>, dim3(grid), dim3(256), 0, st, (bf16*)out, ldo, (const bf16*)ep.bias, ep.act, M, N, (const bf16*)ep.gate, ep.gate_rows, ep.ld_gate, (const bf16*)ep.resid, ep.ld_resid);
  else hipLaunchKernelGGL(bias_act_kernel<float>, dim3(grid), dim3(256), 0, st, (float*)out, ldo, (const float*)ep.bias, ep.act, M, N, (const float*)ep.gate, ep.gate_rows, ep.ld_gate, (const float*)ep.resid, ep.ld_resid);
  BLR_CHECK_LAUNCH("bias_act");
  return BLR_OK;
}

// out[m][c] = silu(y[m][c] + bias[c]) * (y[m][c + h] + bias[c + h]) over a full-width result y (M, 2 h): the gated unit of
// Llama's MLP where no kernel fuses it.  Rounding points as in the fused form: both factors are rounded to T, then their product.
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ y, int64_t ldy, const T* __restrict__ bias, T* __restrict__ out, int64_t ldo, int M, int h) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * h) return;
  const int m = (int)(idx / h), c = (int)(idx - (int64_t)m * h);
  float g = TypeTraits<T>::to_f32(y[(int64_t)m * ldy + c]), u = TypeTraits<T>::to_f32(y[(int64_t)m * ldy + c + h]);
  if (bias) { g += TypeTraits<T>::to_f32(bias[c]); u += TypeTraits<T>::to_f32(bias[c + h]); }
  const T gt = TypeTraits<T>::from_f32(apply_act(g, BLR_ACT_SILU)), ut = TypeTraits<T>::from_f32(u);
  out[(int64_t)m * ldo + c] = TypeTraits<T>::from_f32(TypeTraits<T>::to_f32(gt) * TypeTraits<T>::to_f32(ut));
}

static int silu_mul_launch(const void* y, int64_t ldy, const void* bias, void* out, int64_t ldo, int M, int h, int dtype, hipStream_t st) {
  const unsigned grid = (unsigned)cdiv((int64_t)M * h, 256);
  if (dtype == BLR_F16) hipLaunchKernelGGL(silu_mul_kernel<f16>, dim3(grid), dim3(256), 0, st, (const f16*)y, ldy, (const f16*)bias, (f16*)out, ldo, M, h);
  else if (dtype == BLR_BF16) hipLaunchKernelGGL(silu_mul_kernel<bf16>, dim3(grid), dim3(256), 0, st, (const bf16*)y, ldy, (const bf16*)bias, (bf16*)out, ldo, M, h);
  else hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(grid), dim3(256), 0, st, (const float*)y, ldy, (const float*)bias, (float*)out, ldo, M, h);
  BLR_CHECK_LAUNCH("silu_mul");
  return BLR_OK;
}

// BLR_ACT_SILU_MUL is fused into the write-out of the last GEMM (pairs of tiles) for BLAST with an even number of blocks, low
// rank and dense above 128 rows of f16 / bf16; everything else computes the full-width result into the tail of the workspace
// and finishes with silu_mul_kernel.
static bool silu_mul_fused(int op, int M, int out_f, int dtype, int b) {
  if (dtype == BLR_F32 || M <= 128 || out_f % 16) return false;
  if (op == BLR_OP_BLAST) return b % 2 == 0;
  return op == BLR_OP_LOW_RANK || op == BLR_OP_DENSE;
}
static size_t silu_mul_scratch(int op, int M, int out_f, int dtype, int b) {
  return silu_mul_fused(op, M, out_f, dtype, b) ? 0 : align_up((size_t)M * out_f * elt_size(dtype), 256);
}

// Runs `call(out, ldo, ws_bytes)` (a plain entry point) with the epilogue armed and finishes whatever the call did not fuse.
struct GateResidual { const void* gate; int gate_rows; int64_t ld_gate; const void* resid; int64_t ld_resid; };
template <typename F>
static int with_epilogue(int op, int b, const void* bias, int act, void* out, int64_t ldo, int M, int out_f, int dtype, void* ws, size_t ws_bytes,
                         void* stream, F&& call, GateResidual gr = {nullptr, 0, 0, nullptr, 0}) {
  if (act < BLR_ACT_NONE || act > BLR_ACT_SILU_MUL) { set_error("epilogue: unknown activation %d", act); return BLR_ERR_BAD_ARG; }
  if (act == BLR_ACT_SILU_MUL) {
    if (gr.gate || gr.resid) { set_error("epilogue: BLR_ACT_SILU_MUL takes no gate and no residual"); return BLR_ERR_BAD_ARG; }
    if (M <= 0 || out_f <= 0 || out_f % 2) { set_error("epilogue: BLR_ACT_SILU_MUL needs an even out_f (gate | up)"); return BLR_ERR_BAD_SHAPE; }
    if (!out || ldo < out_f / 2) { set_error("epilogue: out of BLR_ACT_SILU_MUL has out_f / 2 columns; ldo too small"); return BLR_ERR_BAD_ARG; }
    if (!dtype_ok(dtype)) { set_error("epilogue: bad dtype"); return BLR_ERR_BAD_ARG; }
    const size_t extra = silu_mul_scratch(op, M, out_f, dtype, b);
    if (extra) {                                        // full-width result in the tail of the workspace, then the elementwise kernel
      if (!ws || ws_bytes < extra) { set_error("epilogue: BLR_ACT_SILU_MUL needs blr_ep_workspace_bytes() = %zu more bytes of workspace here", extra); return BLR_ERR_WORKSPACE; }
      void* full = reinterpret_cast<char*>(ws) + (ws_bytes - extra) / 256 * 256;
      tl_ep = {nullptr, 0, false, false, nullptr, 0, 0, nullptr, 0};
      const int rc = call(full, (int64_t)out_f, (ws_bytes - extra) / 256 * 256);
      if (rc != BLR_OK) return rc;
      return silu_mul_launch(full, out_f, bias, out, ldo, M, out_f / 2, dtype, (hipStream_t)stream);
    }
    tl_ep = {bias, act, true, false, nullptr, 0, 0, nullptr, 0};
    const int rc = call(out, ldo, ws_bytes);
    const bool used = tl_ep.used;
    tl_ep = {nullptr, 0, false, false, nullptr, 0, 0, nullptr, 0};
    if (rc == BLR_OK && !used) { set_error("epilogue: BLR_ACT_SILU_MUL was not applied (internal error)"); return BLR_ERR_UNSUPPORTED; }
    return rc;
  }
  if (gr.gate && (gr.gate_rows <= 0 || gr.ld_gate < out_f)) { set_error("epilogue: gate needs gate_rows > 0 and ld_gate >= out_f"); return BLR_ERR_BAD_ARG; }
  if (gr.resid && gr.ld_resid < out_f) { set_error("epilogue: ld_resid < out_f"); return BLR_ERR_BAD_ARG; }
  const PendingEpilogue ep = {bias, act, bias != nullptr || act != BLR_ACT_NONE || gr.gate != nullptr || gr.resid != nullptr, false,
                              gr.gate, gr.gate_rows, gr.ld_gate, gr.resid, gr.ld_resid};
  tl_ep = ep;
  const int rc = call(out, ldo, ws_bytes);
  const bool used = tl_ep.used, armed = tl_ep.armed;
  tl_ep = {nullptr, 0, false, false, nullptr, 0, 0, nullptr, 0};
  if (rc != BLR_OK || !armed || used) return rc;
  return bias_act_launch(out, ldo, ep, M, out_f, dtype, (hipStream_t)stream);
}

}  // namespace blr

using namespace blr;

namespace blr {
namespace {
constexpr int kOptUnset = -2147483647 - 1;
const char* const kOptNames[OPT_COUNT] = {"BLR_GEMM_RING", "BLR_GEMM_RING_TILE", "BLR_GEMM_RING_PER_CU", "BLR_GEMM_RING_WAVES", "BLR_GEMM_RING_BK", "BLR_GEMM_SPLITK",
                                          "BLR_DECODE2", "BLR_DECODE3", "BLR_DECODE_PAIR", "BLR_DECODE_ROWS", "BLR_DENSE_SLAB", "BLR_DENSE_ROWS",
                                          "BLR_BLAST_MIXU", "BLR_BLAST_ONE", "BLR_BLAST_YMIXW"};
// what each option may be set to: a range, or (BLR_GEMM_RING_TILE, BLR_GEMM_RING_WAVES) a short list; anything else is refused
bool opt_value_ok(int id, int v) {
  switch (id) {
    case OPT_GEMM_RING: case OPT_GEMM_RING_PER_CU: case OPT_DECODE_PAIR: case OPT_BLAST_MIXU: return v >= 0 && v <= 2;
    case OPT_GEMM_RING_TILE: return v == 0 || v == 256256 || v == 256128 || v == 256096 || v == 128128;
    case OPT_GEMM_RING_WAVES: return v == 4 || v == 8;
    case OPT_GEMM_RING_BK: return v == 32 || v == 64;
    default: return v == 0 || v == 1;
  }
}
std::atomic<int> g_opts[OPT_COUNT];
std::once_flag g_opts_once;
void opts_init() {
  for (int i = 0; i < OPT_COUNT; ++i) {
    const char* e = getenv(kOptNames[i]);
    g_opts[i].store(e && opt_value_ok(i, atoi(e)) ? atoi(e) : kOptUnset, std::memory_order_relaxed);   // (a value out of range is ignored)
  }
}
}  // namespace
int option_value(int id, int dflt) {
  std::call_once(g_opts_once, opts_init);
  const int v = g_opts[id].load(std::memory_order_relaxed);
  return v == kOptUnset ? dflt : v;
}
static std::atomic<unsigned> g_spin_limit{0};
unsigned spin_limit_now() {
  const unsigned v = g_spin_limit.load(std::memory_order_relaxed);
  return v ? v : 4000000u;
}
}  // namespace blr

extern "C" {

void blr_set_spin_limit(unsigned polls) { blr::g_spin_limit.store(polls, std::memory_order_relaxed); }

int blr_set_option(const char* name, int value, int unset) {
  std::call_once(blr::g_opts_once, blr::opts_init);
  for (int i = 0; name && i < blr::OPT_COUNT; ++i)
    if (!strcmp(name, blr::kOptNames[i])) {
      if (!unset && !blr::opt_value_ok(i, value)) { set_error("set_option: %d is not a value of %s", value, name); return BLR_ERR_BAD_ARG; }
      blr::g_opts[i].store(unset ? blr::kOptUnset : value, std::memory_order_relaxed);
      return BLR_OK;
    }
  set_error("set_option: unknown option %s", name ? name : "(null)");
  return BLR_ERR_BAD_ARG;
}

// Synchronises the stream, reads the error word of a streaming workspace and clears it.
int blr_workspace_status(void* ws, size_t ws_bytes, void* stream) {
  if (!ws || ws_bytes < stream_ws_prefix_bytes()) { set_error("workspace_status: not a streaming workspace (%zu bytes)", ws_bytes); return BLR_ERR_WORKSPACE; }
  hipStream_t st = (hipStream_t)stream;
  unsigned* word = reinterpret_cast<unsigned*>(reinterpret_cast<char*>(ws) + stream_ws_error_offset());
  unsigned host = 0;
  hipError_t e = hipMemcpyAsync(&host, word, sizeof(unsigned), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) { set_error("workspace_status: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  if (!host) return BLR_OK;
  e = hipMemsetAsync(word, 0, sizeof(unsigned), st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) { set_error("workspace_status: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
  set_error("a bounded wait inside a kernel gave up since the last query: the results of the calls on this workspace since then are not valid "
            "(another kernel kept part of the GPU busy, or two calls shared the workspace)");
  return BLR_ERR_TIMEOUT;
}

const char* blr_last_error(void) { return g_err; }
int blr_version(void) { return 100; }
int blr_device_cus(void) { return device_cus(); }

static int resolve_algo(int algo, int M, int dtype, bool want_intermediates) {
  if (algo == BLR_ALGO_AUTO) {
    if (dtype != BLR_F32 && M <= 16 && !want_intermediates) return BLR_ALGO_STREAM;
    return BLR_ALGO_TILED;
  }
  return algo;
}

// ---- BLAST ------------------------------------------------------------------------------------
size_t blr_blast_workspace_bytes(int M, int in_f, int out_f, int b, int r, int dtype, int algo) {
  if (M <= 0 || b <= 0 || r <= 0) return 0;
  int a = resolve_algo(algo, M, dtype, false);
  size_t tiled = 2 * align_up((size_t)b * M * r * elt_size(dtype), 256);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    size_t s = stream_blast_workspace(M, in_f, out_f, b, r, 16);
    return s > tiled ? s : tiled;
  }
  return tiled;
}

static int check_blast_shape(const char* who, int M, int in_f, int out_f, int b, int r) {
  if (M <= 0 || in_f <= 0 || out_f <= 0 || b <= 0 || r <= 0) { set_error("%s: non-positive size", who); return BLR_ERR_BAD_ARG; }
  if (b == 1) { set_error("%s: b must not be 1", who); return BLR_ERR_BAD_SHAPE; }   // reference blast_funcs.py:34
  if (in_f % b || out_f % b) { set_error("%s: in_f=%d / out_f=%d not divisible by b=%d", who, in_f, out_f, b); return BLR_ERR_BAD_SHAPE; }
  return BLR_OK;
}

// Three launches: Y = x_j V_j (batched GEMM), Z = mix(S, Y), out_i = Z_i U_i (batched GEMM).  sat8 rounds and
// saturates Y and Z to the int8 range.  Y and Z (b, M, r) live in the workspace unless the caller wants them.
static int blast_tiled(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                       void* out, int64_t ldo, void* z_out, void* y_out,
                       int M, int in_f, int out_f, int b, int r,
                       int dtype, int u_layout, int s_layout, int sat8,
                       void* ws, size_t ws_bytes, hipStream_t st, int fused = 0) {   // fused: 1 = must, 0 = where it applies, -1 = never
  const int P = in_f / b, Q = out_f / b;
  const size_t es = elt_size(dtype);
  const size_t ybytes = align_up((size_t)b * M * r * es, 256);
  size_t need = (y_out ? 0 : ybytes) + (z_out ? 0 : ybytes);
  if (need && (!ws || ws_bytes < need)) { set_error("blast: workspace %zu < %zu", ws_bytes, need); return BLR_ERR_WORKSPACE; }
  char* wp = reinterpret_cast<char*>(ws);
  void* Y = y_out ? y_out : (void*)wp; if (!y_out) wp += ybytes;
  void* Z = z_out ? z_out : (void*)wp;

  int64_t si, sj, sr;
  if (s_layout == BLR_S_JIR) { sj = (int64_t)b * r; si = r; sr = 1; }
  else if (s_layout == BLR_S_RIJ) { sr = (int64_t)b * b; si = b; sj = 1; }
  else { si = (int64_t)b * r; sj = r; sr = 1; }
  int rc = 1;
  int mixu_prepared = 0;
  // A few dozen rows are still a weight-streaming problem: 256-row tiles would leave most compute units without one and the
  // others with a long stream each (4096 -> 4096 at 17 rows: 36 us through the tiles, 12 us at 16 rows through the few-row
  // kernels).  Up to 128 rows the three launches of the few-row path run over tiles of 16 rows with the weights held in registers
  // (at 128 rows 32 / 44 / 43 us against 39 / 48 / 56 us through the tiles on the three Llama-7B layers).
  constexpr int rows_max_m = 128;
  if (M <= rows_max_m && !y_out && !z_out && !sat8 && fused <= 0 && dtype != BLR_F32 && !silu_mul_armed()) {
    StreamBlastArgs s = {};
    s.x = x; s.ldx = ldx; s.U = U; s.V = V; s.S = S; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = r;
    s.dtype = dtype; s.u_layout = u_layout; s.s_layout = s_layout; s.wbits = 16;
    rc = decode_rows_launch(s, ws, ws_bytes, st);
    if (rc != 1) return rc;
  }
  // Nobody asked for Y: x V and the mix can run as one launch with Y kept inside the compute units (BLR_ALGO_FUSED).  Chosen
  // by itself only for narrow input blocks: the fused kernel re-reads V once per 32 rows, and from about 128 columns per
  // block on that costs more than the round trip of Y it saves (measured at 4096 rows: 1152 -> 1152, r = 288: 64 against
  // 68 us; 4608 -> 1152, r = 576: 154 against 122 us; Llama-7B gate_up at 2048 rows: 201 against 186 us).
  constexpr int fuse_max_p = 128;
  // Narrow output blocks (either layout of U: it is re-laid for the kernel anyway): the mix and the product with U run as one launch that reads Y once and
  // never writes Z (blast_mixu_kernel); the first half is then the plain GEMM, which leaves Y.  Measured at 4096 rows against the
  // mix kernel + batched GEMM: 4608 -> 1152, r = 576: 90 against 122 us; against the fused first half + batched GEMM: 1152 -> 1152,
  // r = 288: 47 against 51 us.  BLR_BLAST_MIXU: 0 never, 1 only where the first half would not be fused anyway, 2 (default)
  // wherever the kernel takes the shape.
  const int mixu_mode = option_value(OPT_BLAST_MIXU, 2);
  const bool mixu_shape = !z_out && !sat8 && fused <= 0 && dtype != BLR_F32 && b == 16 && Q % 8 == 0 && Q <= 80 && r % 32 == 0 && !silu_mul_armed();
  // Narrow input blocks as well (at most 96 columns): the whole call is one launch that forms Y per step of the rank walk in the
  // compute unit and keeps neither Y nor Z in memory (blast_one_kernel).  BLR_BLAST_ONE=0 switches it off.
  const int one_mode = option_value(OPT_BLAST_ONE, 1);
  if (one_mode && mixu_shape && !y_out && P <= 96 && P % 8 == 0) {
    GemmArgs e1 = {};
    attach_epilogue_peek(e1);
    rc = blast_one_launch(x, ldx, U, V, S, out, ldo, e1, M, in_f, b, r, Q, si, sj, sr, dtype, ws, ws_bytes, st, u_layout == BLR_U_RQ);
    if (rc == BLR_OK && !sat8) { GemmArgs claim = {}; attach_epilogue(claim); }
    if (rc != 1) return rc;
    rc = 1;
  }
  const bool mixu = mixu_shape && (mixu_mode >= 2 || (mixu_mode == 1 && (P > fuse_max_p || fused < 0)));
  // Wide input blocks (16 of them, a multiple of 64 columns each, rank a multiple of 64): x V as one GEMM whose 64 x 64 tile keeps Y
  // of all 16 blocks in registers, then the mix, in one launch (blast_ymixw_kernel) - by itself from half a round of tiles on
  // (whole calls, before -> after: 4096 -> 4096, r = 512 at 1024 / 2048 / 4096 rows 47.1 -> 46.1 / 65.7 -> 56.3 / 101.9 -> 96.2 us,
  // at 512 rows 40.1 -> 44.3; 4096 -> 22016, r = 1024 at 512 / 1024 / 2048 / 4096 rows 78.6 -> 77.7 / 114.4 -> 104.3 / 179.5 -> 174.0 /
  // 350.6 -> 344.2 us, at 256 rows 55.2 -> 59.3).  BLR_BLAST_YMIXW=0 switches it off; BLR_ALGO_FUSED asks for it at any row count.
  const int cus_now = device_cus() > 0 ? device_cus() : 256;
  const bool ymixw_fill = cdiv(M, 64) * (int64_t)(r / 64) * 2 >= cus_now;
  if (!mixu && !y_out && !sat8 && fused >= 0 && P > fuse_max_p && option_value(OPT_BLAST_YMIXW, 1) && (fused == 1 || ymixw_fill))
    rc = blast_ymixw_launch(x, ldx, V, S, Z, M, in_f, b, r, si, sj, sr, s_layout, dtype, Y, ybytes, st);
  if (rc < 0) return rc;
  if (rc == 1 && !mixu && !y_out && !sat8 && fused >= 0 && (fused == 1 || P <= fuse_max_p))
    rc = blast_ymix_launch(x, ldx, V, S, Z, M, in_f, b, r, si, sj, sr, s_layout, dtype, Y, ybytes, st);   // (the unused room of Y holds S transposed)
  if (rc < 0) return rc;
  if (rc == 1 && fused == 1) { set_error("blast: the fused kernel does not take this shape (b even and <= 16, block width and rank multiples of 8, f16/bf16)"); return BLR_ERR_UNSUPPORTED; }
  if (rc == 1) {
    GemmArgs g1 = {};
    g1.A = x; g1.lda = ldx; g1.sA = P;
    g1.B = V; g1.ldb = r; g1.sB = (int64_t)P * r; g1.b_kn = 1;
    g1.C = Y; g1.ldc = r; g1.sC = (int64_t)M * r; g1.cn = 1;
    g1.M = M; g1.N = r; g1.K = P; g1.batch = b;
    g1.sat8 = sat8;
    if (mixu) {                                     // the GEMM's launch also re-lays U and S for the kernel that follows, if it can
      GemmArgs e2 = {};
      attach_epilogue_peek(e2);
      if (blast_mixu_plan(Y, S, U, out, ldo, e2, M, b, r, Q, si, sj, sr, dtype, Z, ybytes, &g1.side, u_layout == BLR_U_RQ)) g1.side_taken = &mixu_prepared;
      else g1.side.items = 0;
    }
    rc = gemm_launch(g1, dtype, st);
    if (rc) return rc;
    if (!mixu) {
      rc = blast_mix_launch(Y, S, Z, M, b, r, si, sj, sr, dtype, st, sat8);
      if (rc) return rc;
    }
  }

  GemmArgs g2 = {};
  g2.A = Z; g2.lda = r; g2.sA = (int64_t)M * r;
  g2.B = U;
  if (u_layout == BLR_U_RQ) { g2.b_kn = 1; g2.ldb = Q; g2.sB = (int64_t)r * Q; }
  else { g2.b_kn = 0; g2.ldb = r; g2.sB = (int64_t)Q * r; }
  g2.C = out; g2.ldc = ldo; g2.sC = Q; g2.cn = 1;
  g2.M = M; g2.N = Q; g2.K = r; g2.batch = b;
  if (!sat8) attach_epilogue(g2);
  if (g2.pair) {                                    // silu(gate) * up: output blocks i and i + b/2 as the two tiles of a work item
    if (sat8 || b % 2) { set_error("blast: BLR_ACT_SILU_MUL needs an even number of blocks"); return BLR_ERR_UNSUPPORTED; }
    g2.batch = b / 2; g2.pair_dA = (int64_t)(b / 2) * g2.sA; g2.pair_dB = (int64_t)(b / 2) * g2.sB; g2.pair_dbias = (int64_t)(b / 2) * Q;
  }
  if (mixu) {                                       // (Y is in memory: the branch above ran the GEMM and skipped the mix)
    rc = blast_mixu_launch(Y, S, U, out, ldo, g2, M, b, r, Q, si, sj, sr, s_layout, dtype, Z, ybytes, st, mixu_prepared != 0, u_layout == BLR_U_RQ);
    if (rc != 1) return rc;
    rc = blast_mix_launch(Y, S, Z, M, b, r, si, sj, sr, dtype, st, sat8);
    if (rc) return rc;
  }
  return gemm_launch(g2, dtype, st);
}

int blr_blast_fwd(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                  void* out, int64_t ldo, void* z_out, void* y_out,
                  int M, int in_f, int out_f, int b, int r,
                  int dtype, int u_layout, int s_layout, int algo,
                  void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!x || !U || !V || !S || !out) { set_error("blast: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype) || u_layout < 0 || u_layout > 1 || s_layout < 0 || s_layout > 2) { set_error("blast: bad enum"); return BLR_ERR_BAD_ARG; }
  int rc = check_blast_shape("blast", M, in_f, out_f, b, r);
  if (rc) return rc;
  if (ldx < in_f || ldo < (silu_mul_armed() ? out_f / 2 : out_f)) { set_error("blast: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  const int P = in_f / b, Q = out_f / b;
  int a = resolve_algo(algo, M, dtype, z_out || y_out);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    if (dtype == BLR_F32 || M > 16 || z_out || y_out) { set_error("blast: streaming algorithm needs f16/bf16, M <= 16, no intermediates"); return BLR_ERR_UNSUPPORTED; }
    StreamBlastArgs s = {};
    s.x = x; s.ldx = ldx; s.U = U; s.V = V; s.S = S; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = r;
    s.dtype = dtype; s.u_layout = u_layout; s.s_layout = s_layout; s.wbits = 16;
    s.ws = ws; s.ws_bytes = ws_bytes; s.split = (a == BLR_ALGO_STREAM_SPLIT);
    return stream_blast_launch(s, st);
  }
  if (a != BLR_ALGO_TILED && a != BLR_ALGO_FUSED) { set_error("blast: algorithm %d not available", a); return BLR_ERR_UNSUPPORTED; }
  if (a == BLR_ALGO_FUSED && y_out) { set_error("blast: the fused algorithm never forms Y in memory (y_out must be null)"); return BLR_ERR_UNSUPPORTED; }
  return blast_tiled(x, ldx, U, V, S, out, ldo, z_out, y_out, M, in_f, out_f, b, r, dtype, u_layout, s_layout, 0, ws, ws_bytes, st,
                     a == BLR_ALGO_FUSED ? 1 : 0);
}

// ---- BLAST with int8-valued intermediates ----------------------------------------------------------
// Reference triton_funcs/blast_sym_quant_kernels.py:92-112 (Y), :214-234 (Z), :340-360 (out): the two
// intermediates are rounded to nearest even and saturated to [-128, 127] after fp32 accumulation.  The
// values are kept in the activation dtype (every integer of that range is exact in f16, bf16 and f32).
size_t blr_blast_i8act_workspace_bytes(int M, int in_f, int out_f, int b, int r, int dtype) {
  (void)in_f; (void)out_f;
  if (M <= 0 || b <= 0 || r <= 0) return 0;
  return 2 * align_up((size_t)b * M * r * elt_size(dtype), 256);
}

int blr_blast_i8act_fwd(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                        void* out, int64_t ldo, void* z_out, void* y_out,
                        int M, int in_f, int out_f, int b, int r,
                        int dtype, int u_layout, int s_layout,
                        void* ws, size_t ws_bytes, void* stream) {
  if (!x || !U || !V || !S || !out) { set_error("blast_i8act: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype) || u_layout < 0 || u_layout > 1 || s_layout < 0 || s_layout > 2) { set_error("blast_i8act: bad enum"); return BLR_ERR_BAD_ARG; }
  int rc = check_blast_shape("blast_i8act", M, in_f, out_f, b, r);
  if (rc) return rc;
  if (ldx < in_f || ldo < out_f) { set_error("blast_i8act: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  return blast_tiled(x, ldx, U, V, S, out, ldo, z_out, y_out, M, in_f, out_f, b, r, dtype, u_layout, s_layout, 1,
                     ws, ws_bytes, (hipStream_t)stream);
}

// ---- quantized BLAST -----------------------------------------------------------------------------
size_t blr_blast_q_workspace_bytes(int M, int in_f, int out_f, int b, int r, int bits) {
  if (M <= 0 || b <= 0 || r <= 0) return 0;
  // M <= 16 streams the codes (the decode kernels widen them in registers).  Above that the factors are expanded to two-byte
  // values once per call ([kernel workspace][U][V]) and the two-byte kernels run; the size covers both.
  size_t s = stream_blast_workspace(M <= 16 ? M : 16, in_f, out_f, b, r, bits);
  if (M <= 4) return s;
  size_t sub = M <= 16 ? s : 2 * align_up((size_t)b * M * r * 2, 256);
  return align_up(sub, 256) + align_up((size_t)r * out_f * 2, 256) + align_up((size_t)r * in_f * 2, 256);
}

int blr_blast_q_fwd(const void* x, int64_t ldx, const void* u_codes, const void* u_scales,
                    const void* v_codes, const void* v_scales, const void* S,
                    void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                    int dtype, int bits, int algo, void* ws, size_t ws_bytes, void* stream) {
  if (!x || !u_codes || !u_scales || !v_codes || !v_scales || !S || !out) { set_error("blast_q: null pointer"); return BLR_ERR_BAD_ARG; }
  if (bits != 8 && bits != 4) { set_error("blast_q: bits must be 8 or 4"); return BLR_ERR_BAD_ARG; }
  if (dtype != BLR_F16 && dtype != BLR_BF16) { set_error("blast_q: dtype must be f16 or bf16"); return BLR_ERR_UNSUPPORTED; }
  int rc = check_blast_shape("blast_q", M, in_f, out_f, b, r);
  if (rc) return rc;
  if (r % 8) { set_error("blast_q: r=%d must be a multiple of 8", r); return BLR_ERR_BAD_SHAPE; }
  if ((out_f / b) % 8) { set_error("blast_q: out_f / b = %d must be a multiple of 8", out_f / b); return BLR_ERR_BAD_SHAPE; }
  // rows of codes that are not whole 16-byte pieces (r = 1488 at 4 bits: 744 bytes) are served by the three-launch path only,
  // whose lanes fetch 8 columns (8 or 4 bytes) at a time
  const bool whole16 = ((int64_t)r * bits) % 128 == 0 && ((int64_t)(out_f / b) * bits) % 128 == 0;
  if (ldx < in_f || ldo < out_f) { set_error("blast_q: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  if (!aligned(u_codes, 16) || !aligned(v_codes, 16)) { set_error("blast_q: code buffers must be 16-byte aligned"); return BLR_ERR_BAD_ARG; }
  hipStream_t st = (hipStream_t)stream;
  const bool phase_engine = algo == BLR_ALGO_STREAM || algo == BLR_ALGO_STREAM_SPLIT;
  if (M > 16 && phase_engine) { set_error("blast_q: M=%d > 16 not served by the streaming kernel", M); return BLR_ERR_UNSUPPORTED; }
  // codes at 5..16 rows go to the matrix-core decode kernel as they are (it widens them in registers)
  if (M > 16) {
    size_t need = blr_blast_q_workspace_bytes(M, in_f, out_f, b, r, bits);
    if (!ws || ws_bytes < need) { set_error("blast_q: workspace %zu < %zu", ws_bytes, need); return BLR_ERR_WORKSPACE; }
    if (M <= 128) {                                  // and up to 128 rows too, in tiles of 16 rows: no dequantized copy of the weights
      StreamBlastArgs s = {};
      s.x = x; s.ldx = ldx; s.U = u_codes; s.V = v_codes; s.S = S; s.u_scales = u_scales; s.v_scales = v_scales;
      s.out = out; s.ldo = ldo; s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = r;
      s.dtype = dtype; s.u_layout = BLR_U_RQ; s.s_layout = BLR_S_RIJ; s.wbits = bits;
      rc = decode_rows_launch(s, ws, ws_bytes, st);
      if (rc != 1) return rc;
    }
    const size_t sub = align_up(M <= 16 ? stream_blast_workspace(M, in_f, out_f, b, r, bits) : 2 * align_up((size_t)b * M * r * 2, 256), 256);
    char* wp = reinterpret_cast<char*>(ws) + sub;
    void* Ud = wp; wp += align_up((size_t)r * out_f * 2, 256);
    void* Vd = wp;
    // both factors are (k, n)-ordered with one scale per column of their block: U (b, r, q), V (b, p, r)
    const int64_t urows = (int64_t)b * r, vrows = in_f, q = out_f / b;
    if (dtype == BLR_F16) {
      hipLaunchKernelGGL(dequant_kernel<f16>, dim3(2048), dim3(256), 0, st, (const uint8_t*)u_codes, (const f16*)u_scales, (f16*)Ud, urows, q, bits, 1, (int64_t)r);
      hipLaunchKernelGGL(dequant_kernel<f16>, dim3(2048), dim3(256), 0, st, (const uint8_t*)v_codes, (const f16*)v_scales, (f16*)Vd, vrows, (int64_t)r, bits, 1, (int64_t)(in_f / b));
    } else {
      hipLaunchKernelGGL(dequant_kernel<bf16>, dim3(2048), dim3(256), 0, st, (const uint8_t*)u_codes, (const f16*)u_scales, (bf16*)Ud, urows, q, bits, 1, (int64_t)r);
      hipLaunchKernelGGL(dequant_kernel<bf16>, dim3(2048), dim3(256), 0, st, (const uint8_t*)v_codes, (const f16*)v_scales, (bf16*)Vd, vrows, (int64_t)r, bits, 1, (int64_t)(in_f / b));
    }
    BLR_CHECK_LAUNCH("dequant");
    return blr_blast_fwd(x, ldx, Ud, Vd, S, out, ldo, nullptr, nullptr, M, in_f, out_f, b, r, dtype, BLR_U_RQ, BLR_S_RIJ,
                         M <= 16 ? BLR_ALGO_STREAM : BLR_ALGO_TILED, ws, sub, stream);
  }
  StreamBlastArgs s = {};
  s.x = x; s.ldx = ldx; s.U = u_codes; s.V = v_codes; s.S = S; s.u_scales = u_scales; s.v_scales = v_scales;
  s.out = out; s.ldo = ldo; s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = r;
  s.dtype = dtype; s.u_layout = BLR_U_RQ; s.s_layout = BLR_S_RIJ; s.wbits = bits;
  s.ws = ws; s.ws_bytes = ws_bytes; s.split = (algo == BLR_ALGO_STREAM_SPLIT);
  s.rows_only = whole16 ? 0 : 1;
  return stream_blast_launch(s, st);
}

int blr_quantize_sym(const void* w, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                     int bits, void* codes, void* scales, void* stream) {
  if (!w || !codes || !scales) { set_error("quantize: null pointer"); return BLR_ERR_BAD_ARG; }
  if (outer <= 0 || reduce <= 0 || inner <= 0 || (bits != 8 && bits != 4) || !dtype_ok(dtype)) { set_error("quantize: bad argument"); return BLR_ERR_BAD_ARG; }
  if (bits == 4 && ((inner == 1 ? reduce : inner) % 2)) { set_error("quantize: int4 needs an even contiguous axis"); return BLR_ERR_BAD_SHAPE; }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == BLR_F32) return quantize_t<float>(w, outer, reduce, inner, bits, codes, scales, st);
  if (dtype == BLR_F16) return quantize_t<f16>(w, outer, reduce, inner, bits, codes, scales, st);
  return quantize_t<bf16>(w, outer, reduce, inner, bits, codes, scales, st);
}

// ---- Monarch --------------------------------------------------------------------------------------
// Monarch at 17..128 rows through the few-row kernels: bytes of their intermediates - the first product's output (in slices
// of the input blocks when those are deeper than 1024 rows, as decode_rows_launch cuts them) and the permuted z.
static size_t monarch_rows_bytes(int M, int in_f, int b, int rank, int dtype) {
  if (M <= 16 || M > 128 || dtype == BLR_F32 || b < 2 || in_f % b || rank % b) return 0;
  const int P = in_f / b;
  int mks = 1;
  if (P > 1024)
    for (int ks = (P + 1023) / 1024; ks <= 8; ++ks)
      if (P % ks == 0 && (P / ks) % 8 == 0) { mks = ks; break; }
  return align_up((size_t)b * mks * M * rank * (mks > 1 ? 4 : 2), 256) + align_up((size_t)b * M * rank * 2, 256);   // slices: fp32 partial sums
}

size_t blr_monarch_workspace_bytes(int M, int in_f, int out_f, int b, int rank, int dtype, int algo) {
  if (M <= 0 || b <= 0 || rank <= 0) return 0;
  int a = resolve_algo(algo, M, dtype, false);
  size_t tiled = align_up((size_t)b * M * rank * elt_size(dtype), 256);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    size_t s = stream_generic_workspace(2, M, in_f, out_f, b, rank);
    return s > tiled ? s : tiled;
  }
  const size_t rows = monarch_rows_bytes(M, in_f, b, rank, dtype);
  return rows > tiled ? rows : tiled;
}

int blr_monarch_fwd(const void* x, int64_t ldx, const void* w1, const void* w2,
                    void* out, int64_t ldo, void* out1,
                    int M, int in_f, int out_f, int b, int rank,
                    int dtype, int w2_layout, int out_order, int algo,
                    void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!x || !w1 || !w2 || !out) { set_error("monarch: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype) || w2_layout < 0 || w2_layout > 1 || out_order < 0 || out_order > 1) { set_error("monarch: bad enum"); return BLR_ERR_BAD_ARG; }
  if (M <= 0 || in_f <= 0 || out_f <= 0 || b <= 0 || rank <= 0) { set_error("monarch: non-positive size"); return BLR_ERR_BAD_ARG; }
  if (in_f % b || out_f % b || rank % b) { set_error("monarch: in_f, out_f and rank must be divisible by b=%d", b); return BLR_ERR_BAD_SHAPE; }   // reference wrappers.py:13-14
  if (ldx < in_f || ldo < out_f) { set_error("monarch: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  const int P = in_f / b, S = out_f / b, per = rank / b;
  int a = resolve_algo(algo, M, dtype, out1 != nullptr);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    if (dtype == BLR_F32 || M > 16 || out1) { set_error("monarch: streaming algorithm needs f16/bf16, M <= 16, no intermediates"); return BLR_ERR_UNSUPPORTED; }
    StreamGenericArgs s = {};
    s.x = x; s.ldx = ldx; s.W1 = w1; s.W2 = w2; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = rank; s.dtype = dtype; s.op = 2;
    s.w2_layout = w2_layout; s.out_order = out_order; s.ws = ws; s.ws_bytes = ws_bytes; s.split = (a == BLR_ALGO_STREAM_SPLIT);
    return stream_generic_launch(s, st);
  }
  if (a != BLR_ALGO_TILED) { set_error("monarch: algorithm %d not available", a); return BLR_ERR_UNSUPPORTED; }
  if (!out1 && ws && monarch_rows_bytes(M, in_f, b, rank, dtype) && ws_bytes >= monarch_rows_bytes(M, in_f, b, rank, dtype)) {
    StreamBlastArgs bl = {};
    bl.x = x; bl.ldx = ldx; bl.U = w2; bl.V = w1; bl.S = nullptr; bl.out = out; bl.ldo = ldo;
    bl.M = M; bl.in_f = in_f; bl.out_f = out_f; bl.b = b; bl.bo = b; bl.r = rank;
    bl.dtype = dtype; bl.u_layout = w2_layout == BLR_W2_SR ? BLR_U_QR : BLR_U_RQ; bl.s_layout = BLR_S_IJR; bl.wbits = 16;
    bl.perm_per = per;
    if (out_order == BLR_OUT_INTERLEAVED) { bl.out_bs = 1; bl.out_ns = b; }
    else { bl.out_bs = S; bl.out_ns = 1; }
    const int rc = decode_rows_launch(bl, ws, ws_bytes, st);
    if (rc != 1) return rc;
  }
  const size_t need = out1 ? 0 : align_up((size_t)b * M * rank * elt_size(dtype), 256);
  if (need && (!ws || ws_bytes < need)) { set_error("monarch: workspace %zu < %zu", ws_bytes, need); return BLR_ERR_WORKSPACE; }
  void* O1 = out1 ? out1 : ws;

  GemmArgs g1 = {};
  g1.A = x; g1.lda = ldx; g1.sA = P;
  g1.B = w1; g1.ldb = rank; g1.sB = (int64_t)P * rank; g1.b_kn = 1;
  g1.C = O1; g1.ldc = rank; g1.sC = 0; g1.cn = 1;
  g1.epi = EPI_MONARCH_SCATTER; g1.per = per; g1.sL = (int64_t)M * rank;
  g1.M = M; g1.N = rank; g1.K = P; g1.batch = b;
  int rc = gemm_launch(g1, dtype, st);
  if (rc) return rc;

  GemmArgs g2 = {};
  g2.A = O1; g2.lda = rank; g2.sA = (int64_t)M * rank;
  g2.B = w2;
  if (w2_layout == BLR_W2_SR) { g2.b_kn = 0; g2.ldb = rank; g2.sB = (int64_t)S * rank; }
  else { g2.b_kn = 1; g2.ldb = S; g2.sB = (int64_t)rank * S; }
  g2.C = out; g2.ldc = ldo;
  if (out_order == BLR_OUT_INTERLEAVED) { g2.sC = 1; g2.cn = b; }
  else { g2.sC = S; g2.cn = 1; }
  g2.M = M; g2.N = S; g2.K = rank; g2.batch = b;
  attach_epilogue(g2);
  return gemm_launch(g2, dtype, st);
}

// ---- low rank -------------------------------------------------------------------------------------
// Low rank at 17..128 rows through the few-row kernels: BLAST with the input cut into 16 (or 8, 4, 2) slices, one output block
// and S = 1.  Bytes of its intermediates (0 when the shape is not for it); the launch returns 1 when it does not apply.
static int low_rank_slices(int in_f) {
  for (int c = 16; c >= 2; c >>= 1)
    if (in_f % c == 0 && (in_f / c) % 8 == 0) return c;
  return 0;
}
static size_t low_rank_rows_bytes(int M, int in_f, int r, int dtype) {
  const int bi = low_rank_slices(in_f);
  if (M <= 16 || M > 128 || dtype == BLR_F32 || !bi) return 0;
  return align_up((size_t)bi * M * r * 4, 256) + align_up((size_t)M * r * 2, 256);   // fp32 partial sums of the slices, then z
}

size_t blr_low_rank_workspace_bytes(int M, int in_f, int out_f, int r, int dtype, int algo) {
  if (M <= 0 || r <= 0) return 0;
  int a = resolve_algo(algo, M, dtype, false);
  size_t tiled = align_up((size_t)M * r * elt_size(dtype), 256);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    size_t s = stream_generic_workspace(1, M, in_f, out_f, 1, r);
    return s > tiled ? s : tiled;
  }
  size_t need = tiled + gemm_splitk_bytes(M, r, in_f, dtype);   // x.A has few output tiles and a long reduction: room to cut it along K
  const size_t rows = low_rank_rows_bytes(M, in_f, r, dtype);   // 17..128 rows: the few-row path (x A in up to 16 slices of the input)
  return rows > need ? rows : need;
}

int blr_low_rank_fwd(const void* x, int64_t ldx, const void* A, const void* B,
                     void* out, int64_t ldo, void* z_out,
                     int M, int in_f, int out_f, int r, int dtype, int algo,
                     void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!x || !A || !B || !out) { set_error("low_rank: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype)) { set_error("low_rank: bad dtype"); return BLR_ERR_BAD_ARG; }
  if (M <= 0 || in_f <= 0 || out_f <= 0 || r <= 0) { set_error("low_rank: non-positive size"); return BLR_ERR_BAD_ARG; }
  if (ldx < in_f || ldo < (silu_mul_armed() ? out_f / 2 : out_f)) { set_error("low_rank: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  int a = resolve_algo(algo, M, dtype, z_out != nullptr);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    if (dtype == BLR_F32 || M > 16 || z_out) { set_error("low_rank: streaming algorithm needs f16/bf16, M <= 16, no intermediates"); return BLR_ERR_UNSUPPORTED; }
    StreamGenericArgs s = {};
    s.x = x; s.ldx = ldx; s.W1 = A; s.W2 = B; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = 1; s.r = r; s.dtype = dtype; s.op = 1;
    s.ws = ws; s.ws_bytes = ws_bytes; s.split = (a == BLR_ALGO_STREAM_SPLIT);
    return stream_generic_launch(s, st);
  }
  if (a != BLR_ALGO_TILED) { set_error("low_rank: algorithm %d not available", a); return BLR_ERR_UNSUPPORTED; }
  if (!z_out && ws && low_rank_rows_bytes(M, in_f, r, dtype) && ws_bytes >= low_rank_rows_bytes(M, in_f, r, dtype)) {
    StreamBlastArgs bl = {};
    bl.x = x; bl.ldx = ldx; bl.U = B; bl.V = A; bl.S = nullptr; bl.out = out; bl.ldo = ldo;
    bl.M = M; bl.in_f = in_f; bl.out_f = out_f; bl.b = low_rank_slices(in_f); bl.bo = 1; bl.r = r;
    bl.dtype = dtype; bl.u_layout = BLR_U_RQ; bl.s_layout = BLR_S_IJR; bl.wbits = 16;
    const int rc = decode_rows_launch(bl, ws, ws_bytes, st);
    if (rc != 1) return rc;
  }
  const size_t need = z_out ? 0 : align_up((size_t)M * r * elt_size(dtype), 256);
  if (need && (!ws || ws_bytes < need)) { set_error("low_rank: workspace %zu < %zu", ws_bytes, need); return BLR_ERR_WORKSPACE; }
  void* Z = z_out ? z_out : ws;
  GemmArgs g1 = {};
  g1.A = x; g1.lda = ldx; g1.B = A; g1.ldb = r; g1.b_kn = 1;
  g1.C = Z; g1.ldc = r; g1.cn = 1; g1.M = M; g1.N = r; g1.K = in_f; g1.batch = 1;
  const size_t tiled = align_up((size_t)M * r * elt_size(dtype), 256);
  if (ws && ws_bytes > tiled) { g1.splitk_ws = static_cast<char*>(ws) + tiled; g1.splitk_bytes = ws_bytes - tiled; }
  int rc = gemm_launch(g1, dtype, st);
  if (rc) return rc;
  GemmArgs g2 = {};
  g2.A = Z; g2.lda = r; g2.B = B; g2.ldb = out_f; g2.b_kn = 1;
  g2.C = out; g2.ldc = ldo; g2.cn = 1; g2.M = M; g2.N = out_f; g2.K = r; g2.batch = 1;
  attach_epilogue(g2);
  if (g2.pair) { g2.N = out_f / 2; g2.pair_dA = 0; g2.pair_dB = out_f / 2; g2.pair_dbias = out_f / 2; }   // columns n and n + out_f / 2 of B
  return gemm_launch(g2, dtype, st);
}

// ---- dense ----------------------------------------------------------------------------------------
size_t blr_dense_workspace_bytes(int M, int in_f, int out_f, int dtype, int algo) {
  if (M <= 0) return 0;
  int a = resolve_algo(algo, M, dtype, false);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) return stream_generic_workspace(0, M, in_f, out_f, 1, 0);
  const size_t rows = dense_rows_bytes(M, in_f, out_f, dtype);      // 17..128 rows: partial products of the slices of the reduction
  const size_t splitk = gemm_splitk_bytes(M, out_f, in_f, dtype);    // more rows, few tiles: fp32 partial sums of the slices of K
  return rows > splitk ? rows : splitk;
}

int blr_dense_fwd(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                  int M, int in_f, int out_f, int dtype, int algo,
                  void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!x || !W || !out) { set_error("dense: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype)) { set_error("dense: bad dtype"); return BLR_ERR_BAD_ARG; }
  if (M <= 0 || in_f <= 0 || out_f <= 0) { set_error("dense: non-positive size"); return BLR_ERR_BAD_ARG; }
  if (ldx < in_f || ldo < (silu_mul_armed() ? out_f / 2 : out_f)) { set_error("dense: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  int a = resolve_algo(algo, M, dtype, false);
  if (a == BLR_ALGO_STREAM || a == BLR_ALGO_STREAM_SPLIT) {
    if (dtype == BLR_F32 || M > 16) { set_error("dense: streaming algorithm needs f16/bf16 and M <= 16"); return BLR_ERR_UNSUPPORTED; }
    StreamGenericArgs s = {};
    s.x = x; s.ldx = ldx; s.W1 = W; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = 1; s.r = 0; s.dtype = dtype; s.op = 0;
    s.ws = ws; s.ws_bytes = ws_bytes; s.split = (a == BLR_ALGO_STREAM_SPLIT);
    return stream_generic_launch(s, st);
  }
  if (a != BLR_ALGO_TILED) { set_error("dense: algorithm %d not available", a); return BLR_ERR_UNSUPPORTED; }
  {
    // 17..128 rows: 256-row tiles would leave most compute units idle and give the others a long stream each (11008 -> 4096
    // at 64 rows: 124 us); the few-row product kernel over tiles of 16 rows instead
    const int rc = dense_rows_launch(x, ldx, W, out, ldo, M, in_f, out_f, dtype, ws, ws_bytes, st);
    if (rc != 1) return rc;
  }
  GemmArgs g = {};
  g.A = x; g.lda = ldx; g.B = W; g.ldb = out_f; g.b_kn = 1;
  g.C = out; g.ldc = ldo; g.cn = 1; g.M = M; g.N = out_f; g.K = in_f; g.batch = 1;
  // few output tiles and a long reduction (11008 -> 4096 at 256 rows: 32 tiles): room to cut it along K
  if (ws && gemm_splitk_bytes(M, out_f, in_f, dtype) && ws_bytes >= gemm_splitk_bytes(M, out_f, in_f, dtype)) { g.splitk_ws = ws; g.splitk_bytes = ws_bytes; }
  attach_epilogue(g);
  if (g.pair) { g.N = out_f / 2; g.pair_dA = 0; g.pair_dB = out_f / 2; g.pair_dbias = out_f / 2; g.splitk_ws = nullptr; g.splitk_bytes = 0; }
  return gemm_launch(g, dtype, st);
}

// ---- fused output stage: out = act(op(x) + bias) ------------------------------------------------------
size_t blr_ep_workspace_bytes(int op, int M, int out_f, int b, int dtype, int act) {
  if (act != BLR_ACT_SILU_MUL || M <= 0 || out_f <= 0 || !dtype_ok(dtype)) return 0;
  return silu_mul_scratch(op, M, out_f, dtype, b);
}

int blr_blast_fwd_ep(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                     void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                     int dtype, int u_layout, int s_layout, int algo,
                     void* ws, size_t ws_bytes, void* stream, const void* bias, int act) {
  return blr_blast_fwd_ep2(x, ldx, U, V, S, out, ldo, M, in_f, out_f, b, r, dtype, u_layout, s_layout, algo, ws, ws_bytes, stream, bias, act,
                           nullptr, 0, 0, nullptr, 0);
}

int blr_monarch_fwd_ep(const void* x, int64_t ldx, const void* w1, const void* w2,
                       void* out, int64_t ldo, int M, int in_f, int out_f, int b, int rank,
                       int dtype, int w2_layout, int out_order, int algo,
                       void* ws, size_t ws_bytes, void* stream, const void* bias, int act) {
  return blr_monarch_fwd_ep2(x, ldx, w1, w2, out, ldo, M, in_f, out_f, b, rank, dtype, w2_layout, out_order, algo, ws, ws_bytes, stream, bias, act,
                             nullptr, 0, 0, nullptr, 0);
}

int blr_low_rank_fwd_ep(const void* x, int64_t ldx, const void* A, const void* B,
                        void* out, int64_t ldo, int M, int in_f, int out_f, int r, int dtype, int algo,
                        void* ws, size_t ws_bytes, void* stream, const void* bias, int act) {
  return blr_low_rank_fwd_ep2(x, ldx, A, B, out, ldo, M, in_f, out_f, r, dtype, algo, ws, ws_bytes, stream, bias, act, nullptr, 0, 0, nullptr, 0);
}

int blr_dense_fwd_ep(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                     int M, int in_f, int out_f, int dtype, int algo,
                     void* ws, size_t ws_bytes, void* stream, const void* bias, int act) {
  return blr_dense_fwd_ep2(x, ldx, W, out, ldo, M, in_f, out_f, dtype, algo, ws, ws_bytes, stream, bias, act, nullptr, 0, 0, nullptr, 0);
}

// ---- the same with a gate and a residual: out = resid + gate[row group] * act(op(x) + bias) -------------------------------------
int blr_blast_fwd_ep2(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                      void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                      int dtype, int u_layout, int s_layout, int algo,
                      void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                      const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid) {
  return with_epilogue(BLR_OP_BLAST, b, bias, act, out, ldo, M, out_f, dtype, ws, ws_bytes, stream, [&](void* o, int64_t ld, size_t wsb) {
    return blr_blast_fwd(x, ldx, U, V, S, o, ld, nullptr, nullptr, M, in_f, out_f, b, r, dtype, u_layout, s_layout, algo, ws, wsb, stream);
  }, {gate, gate_rows, ld_gate, resid, ld_resid});
}

int blr_monarch_fwd_ep2(const void* x, int64_t ldx, const void* w1, const void* w2,
                        void* out, int64_t ldo, int M, int in_f, int out_f, int b, int rank,
                        int dtype, int w2_layout, int out_order, int algo,
                        void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                        const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid) {
  return with_epilogue(BLR_OP_MONARCH, b, bias, act, out, ldo, M, out_f, dtype, ws, ws_bytes, stream, [&](void* o, int64_t ld, size_t wsb) {
    return blr_monarch_fwd(x, ldx, w1, w2, o, ld, nullptr, M, in_f, out_f, b, rank, dtype, w2_layout, out_order, algo, ws, wsb, stream);
  }, {gate, gate_rows, ld_gate, resid, ld_resid});
}

int blr_low_rank_fwd_ep2(const void* x, int64_t ldx, const void* A, const void* B,
                         void* out, int64_t ldo, int M, int in_f, int out_f, int r, int dtype, int algo,
                         void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                         const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid) {
  return with_epilogue(BLR_OP_LOW_RANK, 1, bias, act, out, ldo, M, out_f, dtype, ws, ws_bytes, stream, [&](void* o, int64_t ld, size_t wsb) {
    return blr_low_rank_fwd(x, ldx, A, B, o, ld, nullptr, M, in_f, out_f, r, dtype, algo, ws, wsb, stream);
  }, {gate, gate_rows, ld_gate, resid, ld_resid});
}

int blr_dense_fwd_ep2(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                      int M, int in_f, int out_f, int dtype, int algo,
                      void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                      const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid) {
  return with_epilogue(BLR_OP_DENSE, 1, bias, act, out, ldo, M, out_f, dtype, ws, ws_bytes, stream, [&](void* o, int64_t ld, size_t wsb) {
    return blr_dense_fwd(x, ldx, W, o, ld, M, in_f, out_f, dtype, algo, ws, wsb, stream);
  }, {gate, gate_rows, ld_gate, resid, ld_resid});
}


}  // extern "C"

// ---- BLAST forward that allocates nothing ----------------------------------------------------------------------------
// The intermediates Y and Z (and, at up to four rows, the stage-1 result of the two-launch decode path) live in a
// file-scope device array instead of a caller's workspace.  Host code never uses the array's name as an address: the
// device address is resolved once per device with hipGetSymbolAddress and kept in g_scratch_ptr.
namespace {
constexpr size_t kScratchBytes = BLR_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_for_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) { blr::set_error("blast_fwd_static: no usable current device (%d)", dev); return BLR_ERR_LAUNCH; }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) { blr::set_error("blast_fwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e)); return BLR_ERR_LAUNCH; }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return BLR_OK;
}
}  // namespace

extern "C" {

int blr_blast_fwd_static(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                         void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                         int dtype, int u_layout, int s_layout, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!x || !U || !V || !S || !out) { set_error("blast_fwd_static: null pointer"); return BLR_ERR_BAD_ARG; }
  if (!dtype_ok(dtype) || u_layout < 0 || u_layout > 1 || s_layout < 0 || s_layout > 2) { set_error("blast_fwd_static: bad enum"); return BLR_ERR_BAD_ARG; }
  int rc = check_blast_shape("blast_fwd_static", M, in_f, out_f, b, r);
  if (rc) return rc;
  if (ldx < in_f || ldo < out_f) { set_error("blast_fwd_static: leading dimension too small"); return BLR_ERR_BAD_ARG; }
  const size_t need = 2 * align_up((size_t)b * M * r * elt_size(dtype), 256);
  if (need > kScratchBytes) {
    set_error("blast_fwd_static: the intermediates of this call need %zu bytes, the built-in scratch holds %zu (2 * b * M * r elements); "
              "use blr_blast_fwd with a workspace", need, kScratchBytes);
    return BLR_ERR_WORKSPACE;
  }
  void* ptr = nullptr;
  rc = scratch_for_current_device(&ptr);
  if (rc) return rc;
  if (M <= 4 && dtype != BLR_F32) {
    // Two launches with the stage-1 result in the scratch (plain loads and stores between them, nothing to clear).
    StreamBlastArgs s = {};
    s.x = x; s.ldx = ldx; s.U = U; s.V = V; s.S = S; s.out = out; s.ldo = ldo;
    s.M = M; s.in_f = in_f; s.out_f = out_f; s.b = b; s.r = r;
    s.dtype = dtype; s.u_layout = u_layout; s.s_layout = s_layout; s.wbits = 16;
    rc = decode_pair_launch(s, ptr, kScratchBytes, st);
    if (rc != 1) return rc;
  }
  // Three launches: Y = x V, Z = mix(S, Y), out = Z U; Y and Z are written in full before they are read.
  return blast_tiled(x, ldx, U, V, S, out, ldo, nullptr, nullptr, M, in_f, out_f, b, r, dtype, u_layout, s_layout, 0, ptr, kScratchBytes, st);
}

}  // extern "C"

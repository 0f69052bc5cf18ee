// Device-side helpers shared by the decode kernels (blr_decode.hip, blr_decode3.hip): tagged hand-over values,
// streaming loads through buffer descriptors, the epoch protocol, division by a launch constant.
#pragma once
#include <cstdio>
#include <cstdlib>
#include "blr_common.h"

namespace blr {

constexpr int D2_SHARDS = 16;                 // check-in counters, 256 bytes apart
constexpr unsigned D2_SPIN_LIMIT = 4000000u;  // polls before a bounded wait gives up and sets the error word

__device__ __forceinline__ unsigned long long ld_tag(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_tag(unsigned long long* p, float v, unsigned epoch) {
  __hip_atomic_store(p, ((unsigned long long)epoch << 32) | (unsigned long long)__float_as_uint(v),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16 bytes of weights -> fp32: 8 two-byte elements, 16 int8 codes or 32 int4 codes (low nibble first).
template <typename T, int WB>
__device__ __forceinline__ void cvtw(const u32x4& r, float (&w)[128 / WB]) {
  if constexpr (WB == 16) {
    typename TypeTraits<T>::vec8 v = __builtin_bit_cast(typename TypeTraits<T>::vec8, r);
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = TypeTraits<T>::to_f32(v[e]);
  } else if constexpr (WB == 8) {
#pragma unroll
    for (int e = 0; e < 16; ++e) w[e] = (float)(int8_t)((r[e >> 2] >> ((e & 3) * 8)) & 0xFF);
  } else {
#pragma unroll
    for (int e = 0; e < 32; ++e) w[e] = (float)(((int32_t)(r[e >> 3] << (28 - 4 * (e & 7)))) >> 28);
  }
}
// 16-byte streaming load through a buffer descriptor that spans the whole factor: the per-lane
// byte offset sits in one register, the per-load row offset is uniform (scalar), and a row past
// the end of the factor reads as zero instead of faulting - no clamping, no 64-bit addresses.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wbuf(const void* W, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(W), 0, bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 ldw16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 2));   // nt
}

// Workgroup 0, at its end: wait until every workgroup of the launch has checked in (each does so once it holds its
// copy of the epoch), then publish the epoch of this call, from which the next call derives its own.  The check-in
// counters are never cleared: the word behind them holds the total of all earlier calls, so a wait that gave up
// (the error word is then set) leaves nothing behind that a later call could trip over - the late check-ins of
// that call land before its kernel ends and are part of the total the next call starts from.
__device__ __forceinline__ void finish_epoch(unsigned* arrive_word, unsigned* epoch_word, unsigned* err_word, unsigned epoch, int G,
                                             unsigned spin_limit) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    unsigned* base_word = &arrive_word[D2_SHARDS * 64];
    const unsigned base = __hip_atomic_load(base_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned spins = 0;
    while (true) {
      unsigned v = (lane < D2_SHARDS) ? __hip_atomic_load(&arrive_word[lane * 64], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
#pragma unroll
      for (int o = 1; o < D2_SHARDS; o <<= 1) v += __shfl_xor(v, o, 64);
      if ((unsigned)(__shfl(v, 0, 64) - base) >= (unsigned)G) break;
      if (++spins > spin_limit) {
        if (lane == 0) __hip_atomic_store(err_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (lane == 0) {
      __hip_atomic_store(base_word, base + (unsigned)G, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(epoch_word, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// v + the value of v in another lane of the same row of 16 lanes (DPP control word CTRL)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Workgroup w of a launch runs on XCD w % 8, and each XCD has its own L2.  Item order that gives every XCD a contiguous
// run of the G items: neighbouring items (column chunks of one factor block, whose row pieces share cache lines when they
// are not whole lines) then meet in one L2 instead of fetching the shared lines twice.
__device__ __forceinline__ uint32_t xcd_item(uint32_t w, uint32_t G) {
  const uint32_t x = w & 7u, base = G >> 3, rem = G & 7u;
  return x * base + (x < rem ? x : rem) + (w >> 3);
}

// Division of a small number (< 65536) by a launch constant d (< 65536) without the divide sequence: m = ceil(2^32 / d),
// n / d = high word of n * m; d == 1 is flagged by m == 0.
struct FastDiv { uint32_t d, m; };
__device__ __forceinline__ uint32_t fd_div(uint32_t n, FastDiv f) { return f.m ? __umulhi(n, f.m) : n; }
static inline FastDiv fd_make(uint32_t d) {
  FastDiv f; f.d = d; f.m = d <= 1 ? 0u : (uint32_t)((((uint64_t)1 << 32) + d - 1) / d);
  return f;
}

// ---- host side -------------------------------------------------------------------------------------------------
namespace {
int env_i(const char* name, int dflt) {
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
}
// "this shape is not for me": 1, with the place reported when BLR_D2_DEBUG is set
int d2_bail(int line) {
  static const int dbg = env_i("BLR_D2_DEBUG", 0);
  if (dbg) fprintf(stderr, "decode2: falling back (blr_decode.hip:%d)\n", line);
  return 1;
}
int ilog2(int v) { int l = 0; while ((1 << l) < v) ++l; return l; }
}  // namespace

}  // namespace blr

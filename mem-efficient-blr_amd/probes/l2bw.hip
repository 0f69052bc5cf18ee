// Probe, not part of the library: what the vector memory path of a compute unit delivers from an L2-resident buffer, by the shape
// of a load instruction - 1 KiB contiguous, 16 rows x 64 bytes (a 32-k stage of a K-contiguous GEMM operand), 8 rows x 128 bytes
// (a 64-k stage) - to registers and straight to LDS (global_load_lds_dwordx4), with every compute unit reading at once.
// Build and run:  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops mem-efficient-blr_amd/probes/l2bw.hip -o l2bw && ./l2bw
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// MODE 0: global_load_dwordx4 to registers; 1: global_load_lds_dwordx4; ROWB: bytes a lane group of (ROWB/16) lanes reads contiguously
// (1024 = the wave reads 1 KiB contiguous; 64 = 16 rows of 64 bytes, rows `pitch` bytes apart as in a K-contiguous operand tile)
template <int MODE, int ROWB, int UNROLL>
__global__ __launch_bounds__(512) void k(const char* buf, uint32_t mask, int pitch, int iters, unsigned* sink) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lpr = ROWB / 16;                        // lanes per row
  const uint32_t lane_off = (uint32_t)((lane / lpr) * pitch + (lane % lpr) * 16);
  const uint32_t span = (uint32_t)(64 / lpr) * pitch;   // bytes of address space one instruction covers (rows x pitch)
  uint32_t pos = (blockIdx.x * 8u + wave) * 40503u * 1024u;
  u32x4 x = {0, 0, 0, 0};
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)((void __attribute__((address_space(3)))*)(smem + wave * UNROLL * 1024)));
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
      u32x4 v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t off = ((pos + u * (ROWB == 1024 ? 1024u : 64u) * 977u) & mask) + lane_off;
        v[u] = *reinterpret_cast<const u32x4*>(buf + off);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) x ^= v[u];
    } else {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t off = ((pos + u * (ROWB == 1024 ? 1024u : 64u) * 977u) & mask) + lane_off;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds0 + u * 1024), "v"(off), "s"(buf) : "memory");
      }
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(UNROLL / 2) : "memory");
    }
    pos += 7919u * 1024u;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (MODE == 1) x[0] = reinterpret_cast<unsigned*>(smem)[tid];
  if (x[0] == 0xdeadbeefu && x[1] == 0x12345u) sink[0] = x[2];
  (void)span;
}

template <int MODE, int ROWB, int UNROLL>
void run(const char* name, const char* buf, size_t bytes, int pitch, int waves, int wgs_per_cu, unsigned* sink, hipStream_t st) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = 2000;
  const size_t lds = (size_t)waves * UNROLL * 1024;
  CK(hipFuncSetAttribute((const void*)k<MODE, ROWB, UNROLL>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  const uint32_t span = ROWB == 1024 ? 1024u : (uint32_t)(64 / (ROWB / 16)) * pitch;
  const uint32_t mask = (uint32_t)(bytes / 2 - 1) & ~1023u;         // offsets stay within the first half; rows reach into the rest
  if ((size_t)mask + span + 1024 > bytes) { printf("%s: buffer too small\n", name); return; }
  const int grid = 256 * wgs_per_cu;
  k<MODE, ROWB, UNROLL><<<grid, waves * 64, lds, st>>>(buf, mask, pitch, 50, sink);
  CK(hipEventRecord(e0, st));
  k<MODE, ROWB, UNROLL><<<grid, waves * 64, lds, st>>>(buf, mask, pitch, iters, sink);
  CK(hipEventRecord(e1, st)); CK(hipStreamSynchronize(st));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  const double total = (double)grid * waves * iters * UNROLL * 1024.0;
  printf("%-46s footprint %6.1f MB  waves/CU %2d  in flight/CU %5.0f KB: %7.2f TB/s  (%5.1f KB/us/CU, %4.1f B/clk/CU at 2.4 GHz)\n", name, (mask + 1.0) / 1e6,
         waves * wgs_per_cu, (double)waves * wgs_per_cu * UNROLL, total / (ms * 1e-3) * 1e-12, total / 256 / (ms * 1e3) / 1024, total / 256 / (ms * 1e-3) / 2.4e9);
}

int main() {
  CK(hipSetDevice(0));
  unsigned* sink; CK(hipMalloc(&sink, 64));
  char* buf; const size_t cap = 512u << 20; CK(hipMalloc(&buf, cap)); CK(hipMemset(buf, 1, cap));
  hipStream_t st; CK(hipStreamCreate(&st));
  for (size_t mb : {1, 4, 64}) {
    const size_t bytes = mb << 21;       // mask covers half
    printf("---- offsets within %zu MB\n", mb);
    run<0, 1024, 8>("registers, 1 KiB contiguous, 8 in flight", buf, bytes, 0, 8, 1, sink, st);
    run<0, 1024, 8>("registers, 1 KiB contiguous, 8 in flight", buf, bytes, 0, 8, 2, sink, st);
    run<0, 1024, 16>("registers, 1 KiB contiguous, 16 in flight", buf, bytes, 0, 8, 2, sink, st);
    run<1, 1024, 8>("to LDS, 1 KiB contiguous, 8 in flight", buf, bytes, 0, 8, 1, sink, st);
    run<1, 1024, 16>("to LDS, 1 KiB contiguous, 16 in flight", buf, bytes, 0, 8, 1, sink, st);
    run<1, 1024, 8>("to LDS, 1 KiB contiguous, 8 in flight", buf, bytes, 0, 8, 2, sink, st);
    run<1, 64, 8>("to LDS, 16 rows x 64 B (pitch 8 KiB), 8", buf, bytes, 8192, 8, 1, sink, st);
    run<1, 64, 16>("to LDS, 16 rows x 64 B (pitch 8 KiB), 16", buf, bytes, 8192, 8, 1, sink, st);
    run<1, 128, 16>("to LDS, 8 rows x 128 B (pitch 8 KiB), 16", buf, bytes, 8192, 8, 1, sink, st);
    run<0, 64, 16>("registers, 16 rows x 64 B (pitch 8 KiB), 16", buf, bytes, 8192, 8, 1, sink, st);
  }
  return 0;
}

// Probe, not part of the library: the rate of the matrix instructions under the board's power limit when their operands change with
// every instruction (fragments read from LDS, random fp16 data or all ones): 32 x 32 x 16 against 16 x 16 x 32, same LDS bytes per flop.
// Build and run:  hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops mem-efficient-blr_amd/probes/mfpow.hip -o mfpow && ./mfpow
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// KIND 0: 32x32x16, 8 products per 6 reads (128x64 wave tile); 2: 16x16x32, 32 products (128x64: 8x4 blocks) per 12 reads
// (KIND 1, 16 products per 8 reads on four waves, needs more registers than a 512-thread launch bound leaves and is not run)
template <int KIND, bool ONES>
__global__ __launch_bounds__(512) void k(int iters, unsigned* sink, int waves) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  unsigned h = (tid * 2654435761u) ^ (blockIdx.x * 40503u);
  for (int i = tid; i < 65536 / 2; i += blockDim.x) {
    h ^= h << 13; h ^= h >> 17; h ^= h << 5;
    reinterpret_cast<_Float16*>(smem)[i] = ONES ? (_Float16)1.0f : (_Float16)(((int)(h & 0xffff) - 32768) / 16384.0f);
  }
  __syncthreads();
  const unsigned char* base = smem + (wave & 3) * 8192 + lane * 16;
  uint32_t off = 0;
  float s = 0.f;
  if (KIND < 2) {
    constexpr int TM = 4, TN = KIND == 0 ? 2 : 4;
    f32x16 acc[TM][TN];
    for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
      asm volatile("" : "+v"(off));
      off = (off + 1024) & 8191;                        // the data changes from step to step
      f16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const f16x8*>(base + ((off + i * 1024) & 8191) + 16384);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const f16x8*>(base + ((off + j * 1024) & 8191) + 32768);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) s += acc[i][j][0];
  } else {
    constexpr int TM = 8, TN = 4;
    f32x4 acc[TM][TN];
    for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
      asm volatile("" : "+v"(off));
      off = (off + 1024) & 8191;
      f16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const f16x8*>(base + ((off + i * 1024) & 8191) + 16384);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const f16x8*>(base + ((off + j * 1024) & 8191) + 32768);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    for (int i = 0; i < TM; ++i) for (int j = 0; j < TN; ++j) s += acc[i][j][0];
  }
  if (s == 12345.f) sink[0] = 1;
}

template <int KIND, bool ONES>
void run(const char* name, int waves, unsigned* sink, hipStream_t st) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = 400000;
  CK(hipFuncSetAttribute((const void*)k<KIND, ONES>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  k<KIND, ONES><<<256, waves * 64, 65536, st>>>(1000, sink, waves);
  CK(hipEventRecord(e0, st));
  k<KIND, ONES><<<256, waves * 64, 65536, st>>>(iters, sink, waves);
  CK(hipEventRecord(e1, st)); CK(hipStreamSynchronize(st));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  const double flops_step = KIND == 0 ? 8 * 32768.0 : KIND == 1 ? 16 * 32768.0 : 32 * 16384.0;
  printf("%-64s waves %d: %6.1f%% of 2.5 PFLOP/s\n", name, waves, flops_step * waves * iters * 256 / (ms * 1e-3) / 2.5e15 * 100);
}

int main() {
  CK(hipSetDevice(0));
  unsigned* sink; CK(hipMalloc(&sink, 64));
  hipStream_t st; CK(hipStreamCreate(&st));
  for (int rep = 0; rep < 2; ++rep) {
    run<0, false>("32x32x16, 8 products / 6 fragment reads, random data", 8, sink, st);
    run<2, false>("16x16x32, 32 products / 12 fragment reads, random data", 8, sink, st);
    run<0, true>("32x32x16, 8 products / 6 fragment reads, all ones", 8, sink, st);
    run<2, true>("16x16x32, 32 products / 12 fragment reads, all ones", 8, sink, st);
  }
  return 0;
}

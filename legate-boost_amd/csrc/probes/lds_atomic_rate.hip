// Stand-alone probe, not part of liblbtree.so: the rate of 64-bit LDS atomic adds of one CU in the
// addressing pattern of binned_histogram_kernel's striped sub-histogram (lbt_histogram.hip): 16 waves, a
// lane adds 16 times per row into [bin][column] with 64 columns of 8 bytes, its steps rotated by its lane
// number so that the 16 lanes of a quarter wave meet 16 different bank pairs; E more dependent vector
// instructions per add show how much of the address arithmetic hides behind the LDS.
//
//   make -C legate-boost_amd/csrc probes && ./legate-boost_amd/csrc/probes/lds_atomic_rate
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                               \
  do {                                                      \
    hipError_t e_ = (x);                                    \
    if (e_ != hipSuccess) {                                 \
      printf("%s: %s\n", #x, hipGetErrorString(e_));        \
      exit(1);                                              \
    }                                                       \
  } while (0)

constexpr int kWords = 16384;  // 256 bins x 64 columns

// kPattern 0: rotated steps (no two lanes of a quarter wave in one bank pair); 1: the four rows of a
// quarter wave in the same columns (what the steps would be without the rotation: four lanes per bank
// pair); 2: rotated steps, but the lanes that hold a column in the four quarters of a wave add to one address
template <int E, int kPattern>
__global__ void __launch_bounds__(1024) adds(int iters, unsigned long long* out, unsigned seed)
{
  extern __shared__ unsigned long long s[];
  for (int i = threadIdx.x; i < kWords; i += 1024) s[i] = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  unsigned w[4];
  unsigned x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + seed;
  for (int j = 0; j < 4; j++) {
    x    = x * 1664525u + 1013904223u;
    w[j] = x;
  }
  const unsigned piece = ((lane & 3) * 16) * 8;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      unsigned bin = (w[j >> 2] >> (8 * (j & 3))) & 0xff;
#pragma unroll
      for (int t = 0; t < E; t++) bin = (bin * 3u + w[(j + t) & 3]) & 0xff;
      if (kPattern == 2) bin = j;
      const unsigned column = kPattern == 1 ? j : ((j + lane) & 15);
      const unsigned addr   = (bin << 9) + piece + (column << 3);
      atomicAdd(reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(s) + addr),
                static_cast<unsigned long long>(w[0]) << 32 | w[1]);
    }
    w[it & 3] += it;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = s[5];
}

template <int E, int kPattern>
void run(const char* what, unsigned long long* out)
{
  CK(hipFuncSetAttribute(reinterpret_cast<const void*>(adds<E, kPattern>), hipFuncAttributeMaxDynamicSharedMemorySize,
                         kWords * 8));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  const int iters = 1000;
  float best      = 1e9f;
  for (int rep = 0; rep < 3; rep++) {
    CK(hipEventRecord(a));
    adds<E, kPattern><<<256, 1024, kWords * 8>>>(iters, out, 12345u);
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms;
    CK(hipEventElapsedTime(&ms, a, b));
    if (ms < best) best = ms;
  }
  printf("%-60s %7.3f ms  %5.2f cycles per wave-level add and CU (2.1 GHz)\n", what, best,
         best * 1e-3 * 2.1e9 / (16.0 * iters * 16));
  fflush(stdout);
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
}

int main()
{
  unsigned long long* out;
  CK(hipMalloc(&out, 4096 * 8));
  run<0, 0>("rotated steps, address from one shift-add", out);
  run<1, 0>("  one more dependent vector instruction pair per add", out);
  run<2, 0>("  two more", out);
  run<4, 0>("  four more", out);
  run<0, 1>("no rotation: the four rows of a quarter wave in one bank pair", out);
  run<0, 2>("rotated, the four quarters of a wave on one address", out);
  CK(hipFree(out));
  return 0;
}

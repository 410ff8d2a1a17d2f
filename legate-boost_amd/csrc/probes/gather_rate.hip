// Stand-alone probe, not part of liblbtree.so: the rate at which one MI355X fetches the cache records of
// scattered rows, without any histogram work. It restates the access pattern of binned_histogram_kernel
// below the root (lbt_histogram.hip): a bin cache of n rows x 128 bytes (two 64-byte records per row, one
// per feature group), a sorted list of the rows of the nodes being built (27 % of all rows, as at every
// level of a 10M-row tree), 1024-thread workgroups that walk their share of the list, four lanes per
// record (16 bytes each) and `F` rows per lane in flight. Every line printed is one launch configuration:
// milliseconds (best of 5), records per second, and records per cycle and busy CU at 2.1 GHz.
//
//   make -C legate-boost_amd/csrc probes && ./legate-boost_amd/csrc/probes/gather_rate
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                               \
  do {                                                      \
    hipError_t e_ = (x);                                    \
    if (e_ != hipSuccess) {                                 \
      printf("%s: %s\n", #x, hipGetErrorString(e_));        \
      exit(1);                                              \
    }                                                       \
  } while (0)

// how the workgroups of a launch are paired up
enum Pairing {
  kSingle  = 0,  // every workgroup has a row range of its own and reads the first record of each row
  kSameXcd = 1,  // two workgroups per row range, one per record, both on one XCD (they share its L2)
  kTwoXcds = 2,  // the same two on different XCDs
  kBehind  = 3,  // one XCD, but the second workgroup starts half a range later and wraps round
};

template <int LANES, int F>
__global__ void __launch_bounds__(1024)
  gather(const unsigned char* __restrict__ cache, const int* __restrict__ rows, int n_rows, int pairing, unsigned* out)
{
  int ranges = gridDim.x, range = blockIdx.x, record = 0, shift = 0;
  if (pairing != kSingle) {
    ranges         = gridDim.x / 2;
    const int xcd  = blockIdx.x & 7, slot = blockIdx.x >> 3;  // workgroups go round the 8 XCDs
    range          = pairing == kTwoXcds ? blockIdx.x >> 1 : (slot >> 1) * 8 + xcd;
    record         = pairing == kTwoXcds ? blockIdx.x & 1 : slot & 1;
  }
  const int lo = static_cast<long long>(n_rows) * range / ranges;
  const int hi = static_cast<long long>(n_rows) * (range + 1) / ranges;
  if (pairing == kBehind && record == 1) shift = (hi - lo) / 2;
  const int lane = threadIdx.x % LANES, sub = threadIdx.x / LANES, per_pass = blockDim.x / LANES;
  unsigned acc = 0;
  for (int base = lo; base < hi; base += per_pass * F) {
    uint4 v[F];
#pragma unroll
    for (int u = 0; u < F; u++) {
      int i = base + sub + u * per_pass;
      i     = i < hi ? i : lo;
      if (shift) {
        i += shift;
        if (i >= hi) i -= hi - lo;
      }
      const long long row = rows[i];
      v[u] = *reinterpret_cast<const uint4*>(cache + row * 128 + (LANES == 8 ? 0 : record * 64) + lane * 16);
    }
#pragma unroll
    for (int u = 0; u < F; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u) out[0] = acc;  // keeps the loads alive
}

template <int LANES, int F>
void run(const char* what, const unsigned char* cache, const int* rows, int n_rows, unsigned* out, int grid, int threads,
         int pairing)
{
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  float best = 1e9f;
  for (int rep = 0; rep < 5; rep++) {
    CK(hipEventRecord(e0));
    gather<LANES, F><<<grid, threads>>>(cache, rows, n_rows, pairing, out);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    best = std::min(best, ms);
  }
  const double records = static_cast<double>(n_rows) * (pairing == kSingle ? 1 : 2);
  const int busy       = std::min(grid * threads / 1024, 256);
  printf("%-66s %7.4f ms %7.2f G records/s %6.2f TB/s asked for  %.3f records/cycle/CU\n", what, best,
         records / best / 1e6, records * (LANES == 8 ? 128 : 64) / best / 1e9, records / (best * 1e-3) / 2.1e9 / busy);
  fflush(stdout);
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
}

int main()
{
  const long long n = 10000000;
  unsigned char* cache;
  int* rows;
  unsigned* out;
  CK(hipMalloc(&cache, n * 128));
  CK(hipMemset(cache, 1, n * 128));
  CK(hipMalloc(&out, 64));
  std::vector<int> h;
  unsigned s = 12345;
  for (long long i = 0; i < n; i++) {
    s = s * 1664525u + 1013904223u;
    if ((s >> 8) % 100 < 27) h.push_back(static_cast<int>(i));
  }
  const int n_rows = static_cast<int>(h.size());
  CK(hipMalloc(&rows, n_rows * sizeof(int)));
  CK(hipMemcpy(rows, h.data(), n_rows * sizeof(int), hipMemcpyHostToDevice));
  printf("%d of %lld rows, ascending; cache of %lld x 128 bytes\n", n_rows, n, n);
  run<4, 4>("one 64-byte record per row, 4 rows per lane in flight, 256 x 1024", cache, rows, n_rows, out, 256, 1024, kSingle);
  run<4, 2>("  2 rows per lane in flight", cache, rows, n_rows, out, 256, 1024, kSingle);
  run<4, 8>("  8 rows per lane in flight", cache, rows, n_rows, out, 256, 1024, kSingle);
  run<4, 4>("  1024 workgroups of 256 threads", cache, rows, n_rows, out, 1024, 256, kSingle);
  run<4, 4>("  128 workgroups (half of the CUs)", cache, rows, n_rows, out, 128, 1024, kSingle);
  run<8, 4>("the whole 128-byte line of a row (8 lanes), 256 x 1024", cache, rows, n_rows, out, 256, 1024, kSingle);
  run<8, 4>("  128 workgroups (half of the CUs)", cache, rows, n_rows, out, 128, 1024, kSingle);
  run<4, 4>("both records of a row, two workgroups on one XCD, free running", cache, rows, n_rows, out, 256, 1024, kSameXcd);
  run<4, 4>("  the two on different XCDs", cache, rows, n_rows, out, 256, 1024, kTwoXcds);
  run<4, 4>("  one XCD, the second half a row range behind", cache, rows, n_rows, out, 256, 1024, kBehind);
  CK(hipFree(cache));
  CK(hipFree(rows));
  CK(hipFree(out));
  return 0;
}

// Prints known answers for the pieces of thrust::random that the tree
// learner relies on, using the rocThrust headers of this image on the HOST
// (no GPU, no reference code). Output: JSON on stdout.
//
//   hipcc -std=c++17 -O1 --offload-arch=gfx950 gen_thrust_rng_kat.cpp -o /tmp/gen_kat && /tmp/gen_kat
//
// The three call patterns are the ones at build_tree.cu:114-126 (fresh engine,
// two uniform_real draws) and build_tree.cu:884-887 (fresh engine, discard,
// uniform_int_distribution<int64_t>).
#include <thrust/random.h>
#include <cstdint>
#include <cstdio>
#include <vector>

int main()
{
  std::printf("{\n");
  // 1. two successive uniform_real_distribution<double>(0,1) draws per seed;
  //    the seed is passed as int64 exactly like QuantiseStochasticRounding does
  const int64_t seeds[] = {0, 1, 42, 2147483646LL, 2147483647LL, 2147483648LL, 4294967295LL,
                           4294967296LL, 4294967297LL, -1LL, -2LL, 1234567890123456789LL,
                           -8070450532247928832LL, 0x7fffffffffffffffLL, (int64_t)0x8000000000000000ULL,
                           -6148914691236517206LL, 0x0123456789abcdefLL, -81985529216486896LL, 3000000000LL,
                           -3000000000LL, 987654321987LL, -424242424242LL, 4294967294LL, 2147483649LL};
  std::printf("\"real_pairs\": [\n");
  const int ns = sizeof(seeds) / sizeof(seeds[0]);
  for (int i = 0; i < ns; i++) {
    thrust::default_random_engine eng(seeds[i]);
    thrust::uniform_real_distribution<double> dist(0.0, 1.0);
    double a = dist(eng);
    double b = dist(eng);
    std::printf("  {\"seed\": \"%lld\", \"u1\": \"%a\", \"u2\": \"%a\"}%s\n", (long long)seeds[i], a, b,
                i + 1 < ns ? "," : "");
  }
  std::printf("],\n");
  // 2. sampled rows
  struct Case { int seed; int64_t rows; int n; };
  const Case cases[] = {{0, 100000, 8}, {42, 10000000, 8}, {2147483647, 2, 8}, {1, 1, 4},
                        {123456789, 1000000007LL, 8}, {2147483646, 20000000, 300}};
  std::printf("\"row_samples\": [\n");
  const int nc = sizeof(cases) / sizeof(cases[0]);
  for (int c = 0; c < nc; c++) {
    std::printf("  {\"seed\": %d, \"rows\": %lld, \"out\": [", cases[c].seed, (long long)cases[c].rows);
    for (int idx = 0; idx < cases[c].n; idx++) {
      int seed = cases[c].seed;
      thrust::default_random_engine eng(seed);
      thrust::uniform_int_distribution<int64_t> dist(0, cases[c].rows - 1);
      eng.discard(idx);
      std::printf("%lld%s", (long long)dist(eng), idx + 1 < cases[c].n ? ", " : "");
    }
    std::printf("]}%s\n", c + 1 < nc ? "," : "");
  }
  std::printf("],\n");
  // 3. raw engine stream
  std::printf("\"raw\": [");
  thrust::default_random_engine eng(42);
  for (int i = 0; i < 6; i++) std::printf("%u%s", (unsigned)eng(), i < 5 ? ", " : "");
  std::printf("]\n}\n");
  return 0;
}

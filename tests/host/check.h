// Host-side checks of the library's planners (no GPU): every check file includes one
// product source, so that it sees the plan structures and task tables the planner wrote,
// and is compiled for the host only with -fsanitize=address,undefined.  TEST INFRASTRUCTURE.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

struct ConvShape {
  int n, c, h, w, k, s, p, bias, c_out;
};
struct LinShape {
  int n, d_in, d_out, bias;
};
struct BnShape {
  int n, c, h, w;
};
struct Workload {
  std::string name;
  std::vector<ConvShape> convs;
  std::vector<LinShape> linears;
  std::vector<BnShape> bns;
  std::vector<int> factor_dims;   // every Kronecker factor of the configuration
};

extern int g_failures;
#define EXPECT(cond, ...)                                                       \
  do {                                                                          \
    if (!(cond)) {                                                              \
      if (++g_failures <= 40) {                                                 \
        std::fprintf(stderr, "FAILED %s:%d: %s: ", __FILE__, __LINE__, #cond);  \
        std::fprintf(stderr, __VA_ARGS__);                                      \
        std::fprintf(stderr, "\n");                                             \
      }                                                                         \
    }                                                                           \
  } while (0)

// deterministic pseudo-random numbers for the random shape lists
struct Rng {
  unsigned long long s;
  explicit Rng(unsigned long long seed) : s(seed * 2862933555777941757ULL + 3037000493ULL) {}
  unsigned next() {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    return (unsigned)(s >> 33);
  }
  int range(int lo, int hi) { return lo + (int)(next() % (unsigned)(hi - lo + 1)); }
};

// a fake device address: never dereferenced in host-only mode
inline float *fake_ptr(size_t i) { return reinterpret_cast<float *>((uintptr_t)0x100000000ULL + 4096 * i); }

int check_inverse(const std::vector<Workload> &workloads);
int check_cov(const std::vector<Workload> &workloads);
int check_precond(const std::vector<Workload> &workloads);
int check_pack(const std::vector<Workload> &workloads);
int check_elementwise(const std::vector<Workload> &workloads);

// plan_check <workloads file>: runs the planners of the library on the host (option
// host_only: no GPU is touched) over the benchmark configurations' shapes and a few hundred
// random ones, and replays every task table against what it must cover.  Built with
// -fsanitize=address,undefined; exit status 0 only when nothing failed.  TEST INFRASTRUCTURE.
//
// Workloads file, one record per line:
//   workload <name> | conv n c h w k s p bias c_out | linear n d_in d_out bias | bn n c h w | dim d
#include <cstring>
#include <fstream>
#include <sstream>

#include "../../include/kfac_hip.h"
#include "check.h"

int g_failures = 0;

int main(int argc, char **argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: %s <workloads file>\n", argv[0]);
    return 2;
  }
  std::ifstream f(argv[1]);
  if (!f) {
    std::fprintf(stderr, "cannot read %s\n", argv[1]);
    return 2;
  }
  std::vector<Workload> workloads;
  std::string line;
  while (std::getline(f, line)) {
    std::istringstream in(line);
    std::string kind;
    if (!(in >> kind)) continue;
    if (kind == "workload") {
      workloads.emplace_back();
      in >> workloads.back().name;
      continue;
    }
    if (workloads.empty()) {
      std::fprintf(stderr, "record before the first workload line\n");
      return 2;
    }
    Workload &w = workloads.back();
    if (kind == "conv") {
      ConvShape c;
      in >> c.n >> c.c >> c.h >> c.w >> c.k >> c.s >> c.p >> c.bias >> c.c_out;
      w.convs.push_back(c);
    } else if (kind == "linear") {
      LinShape l;
      in >> l.n >> l.d_in >> l.d_out >> l.bias;
      w.linears.push_back(l);
    } else if (kind == "bn") {
      BnShape b;
      in >> b.n >> b.c >> b.h >> b.w;
      w.bns.push_back(b);
    } else if (kind == "dim") {
      int d;
      in >> d;
      w.factor_dims.push_back(d);
    } else {
      std::fprintf(stderr, "unknown record '%s'\n", kind.c_str());
      return 2;
    }
    if (!in) {
      std::fprintf(stderr, "bad record: %s\n", line.c_str());
      return 2;
    }
  }
  if (kfac_option_set("host_only", 1) != KFAC_OK) {
    std::fprintf(stderr, "the library has no host-only mode\n");
    return 2;
  }
  struct {
    const char *name;
    int (*fn)(const std::vector<Workload> &);
  } parts[] = {{"inverse", check_inverse}, {"covariance", check_cov}, {"precondition", check_precond},
               {"pack", check_pack},       {"elementwise", check_elementwise}};
  for (const auto &p : parts) {
    if (argc > 2 && std::strcmp(argv[2], p.name) != 0) continue;
    const int bad = p.fn(workloads);
    std::printf("%-13s %s (%d failures)\n", p.name, bad ? "FAILED" : "ok", bad);
    std::fflush(stdout);
  }
  std::printf("%d workloads, %d failures\n", (int)workloads.size(), g_failures);
  return g_failures ? 1 : 0;
}

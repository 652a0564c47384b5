// Mutation test of the host model (compiled by tests/test_host_fuzz.py with AddressSanitizer and
// UBSan): seeded random edits of two YAML texts go through the parser, and whatever still parses
// goes through the split enumeration, the partition of every preset and the index remap.  The
// process must end normally whatever the text is.
//   host_fuzz <fusion.yaml> <kernels.yaml> <iterations>   (MAXMUT=n: at most n edits per text)
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <random>
#include <sstream>
#include "../hfuse_amd/csrc/fusion_model.h"
using namespace hfuse;
static std::string slurp(const char *p) { std::ifstream f(p); std::ostringstream s; s << f.rdbuf(); return s.str(); }
int main(int argc, char **argv) {
  std::string fus = slurp(argv[1]), ker = slurp(argv[2]);
  int iters = argc > 3 ? atoi(argv[3]) : 100000;
  std::mt19937_64 rng(12345);
  const char alphabet[] = " \n\t:-#'\"[]{}0123456789abcXYZ,.\\|>&*!%@`";
  long ok = 0, bad = 0;
  for (int it = 0; it < iters; it++) {
    std::string f = fus, k = ker;
    std::string &t = (rng() & 1) ? f : k;
    int nm = getenv("MAXMUT") ? 1 + rng() % atoi(getenv("MAXMUT")) : 1 + rng() % 6;
    for (int m = 0; m < nm && !t.empty(); m++) {
      size_t pos = rng() % t.size();
      switch (rng() % 5) {
        case 0: t[pos] = alphabet[rng() % (sizeof alphabet - 1)]; break;
        case 1: t.erase(pos, 1 + rng() % 8); break;
        case 2: t.insert(pos, 1, alphabet[rng() % (sizeof alphabet - 1)]); break;
        case 3: { size_t p2 = rng() % t.size(); size_t len = std::min<size_t>(rng() % 40, t.size() - p2); t.insert(pos, t.substr(p2, len)); } break;
        case 4: { // replace a number by a huge / negative / zero one
          size_t d = t.find_first_of("0123456789", pos);
          if (d != std::string::npos) { const char *vals[] = {"0", "-1", "4294967296", "99999999999999999999", "1e9", "64", "1024", "3"}; size_t e = t.find_first_not_of("0123456789", d); t.replace(d, (e == std::string::npos ? t.size() : e) - d, vals[rng() % 8]); }
        } break;
      }
    }
    Config cfg; std::string err;
    if (!parse_config((rng() % 16 == 0) ? nullptr : f.c_str(), k.c_str(), cfg, err)) { bad++; continue; }
    ok++;
    for (auto &fr : cfg.fusions) {
      if (fr.kernels.size() == 3) {   // the Context's partition among three, every preset and split
        const KernelRow *r3[3] = {cfg.find(fr.kernels[0]), cfg.find(fr.kernels[1]), cfg.find(fr.kernels[2])};
        if (!r3[0] || !r3[1] || !r3[2]) continue;
        for (const char *pn : {"hfuse", "hfuse_lb", "vfuse", "vfuse_lb"}) {
          for (int idx = -2; idx < 12; idx++) {
            Partition part; std::string e3;
            if (make_partition_n(r3, 3, *find_preset(pn), idx, part, e3) == 0)
              for (int h = 0; h < 3; h++) if (part.hi[h] > part.lo[h]) { (void)local_index(part.lo[h], part.lo[h], part.block_dim[h]); (void)local_index(part.hi[h] - 1, part.lo[h], part.block_dim[h]); }
          }
        }
        continue;
      }
      if (fr.kernels.size() != 2) continue;
      const KernelRow *a = cfg.find(fr.kernels[0]), *b = cfg.find(fr.kernels[1]);
      if (!a || !b) continue;
      int ns = num_splits(*a, *b);
      for (const char *pn : {"hfuse", "hfuse_lb", "vfuse", "vfuse_lb"}) {
        const Preset *p = find_preset(pn);
        for (int idx = -2; idx < ns + 1 && idx < 12; idx++) {
          Partition part; std::string e2;
          if (make_partition(*a, *b, *p, idx, 0, part, e2) == 0) {
            for (int h = 0; h < 2; h++) if (part.hi[h] > part.lo[h]) { (void)local_index(part.lo[h], part.lo[h], part.block_dim[h]); (void)local_index(part.hi[h] - 1, part.lo[h], part.block_dim[h]); }
          }
        }
        Partition part; std::string e2;
        (void)make_partition(*a, *b, *p, -1, (int)(rng() % 1200), part, e2);
      }
    }
  }
  printf("ok %ld bad %ld\n", ok, bad);
  return 0;
}

// Allocation-failure injection for the C-ABI's host side: the n-th `operator new` inside a call
// throws std::bad_alloc, for every n until a call needs fewer allocations than that.  Each call
// must come back with HF_OK or HF_ENOMEM -- never terminate, never leak an exception -- and a
// failed call must leave nothing behind that a later, successful call trips over.
//   alloc_fault <fusion.yaml> <kernels.yaml>      prints "config <n1> plan <n2>" (failures survived)
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <new>
#include <sstream>
#include <string>

#include "hfuse_gfx950.h"

static long g_countdown = -1;  // < 0: allocation never fails

void *operator new(std::size_t n) {
  if (g_countdown >= 0 && g_countdown-- == 0) throw std::bad_alloc();
  void *p = std::malloc(n ? n : 1);
  if (!p) throw std::bad_alloc();
  return p;
}
void operator delete(void *p) noexcept { std::free(p); }
void operator delete(void *p, std::size_t) noexcept { std::free(p); }

static std::string slurp(const char *path) {
  std::ifstream in(path, std::ios::binary);
  std::ostringstream ss;
  ss << in.rdbuf();
  return ss.str();
}

template <class Call>
static int sweep(const char *what, Call call) {
  for (long n = 0; n < 100000; n++) {
    g_countdown = n;
    const int rc = call();
    const bool fired = g_countdown < 0;
    g_countdown = -1;
    if (rc != HF_OK && rc != HF_ENOMEM) {
      std::fprintf(stderr, "%s: allocation %ld failed -> rc %d (%s)\n", what, n, rc, hf_last_error());
      std::exit(1);
    }
    if (rc == HF_ENOMEM && !fired) {
      std::fprintf(stderr, "%s: HF_ENOMEM without an injected failure\n", what);
      std::exit(1);
    }
    if (!fired) return (int)n;  // the call needed fewer than n allocations: done
  }
  std::fprintf(stderr, "%s: still allocating after 100000 injected failures\n", what);
  std::exit(1);
}

int main(int argc, char **argv) {
  if (argc != 3) return 2;
  const std::string fusion = slurp(argv[1]), kernels = slurp(argv[2]);
  const int n_cfg = sweep("hf_config_load_text", [&] {
    hf_config *c = nullptr;
    const int rc = hf_config_load_text(fusion.c_str(), kernels.c_str(), &c);
    if (rc == HF_OK) hf_config_free(c);
    else if (c) { std::fprintf(stderr, "config handle set on failure\n"); std::exit(1); }
    return rc;
  });
  hf_config *cfg = nullptr;
  if (hf_config_load_text(fusion.c_str(), kernels.c_str(), &cfg) != HF_OK) return 1;
  const int n_plan = sweep("hf_plan_create", [&] {
    hf_plan *p = nullptr;
    int rc = hf_plan_create(cfg, 0, "hfuse", HF_SPLIT_TABLE, 0, &p);
    if (rc != HF_OK) return rc;
    rc = hf_plan_set_block(p, 128, 192);
    hf_partition part;
    if (rc == HF_OK) rc = hf_plan_partition(p, &part);
    hf_plan_free(p);
    return rc;
  });
  // and the library still works afterwards
  hf_plan *p = nullptr;
  if (hf_plan_create(cfg, 1, "hfuse_lb", 0, 0, &p) != HF_OK) return 1;
  hf_plan_free(p);
  hf_config_free(cfg);
  std::printf("config %d plan %d\n", n_cfg, n_plan);
  return 0;
}

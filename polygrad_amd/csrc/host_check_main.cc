// host_check: drives the device-independent part of the backend -- plan-file loader,
// kernel-graph analysis, index simplifier, renderer, plan-level fusion, coverage analysis
// -- over plan files given on the command line.  Built by `make asan` together with the
// library's host code under AddressSanitizer and UndefinedBehaviorSanitizer (the
// reference builds its own test binary that way, Makefile:4 there), and run by
// tests/test_host_sanitizers.py.  Exit status 0: every file went through without a
// finding; a file that fails to parse is only an error when it is not expected to.
//
//   host_check plan.polyplan ...           every file must load and lower
//   host_check --garbage plan.polyplan ... every file is also fed back truncated and with
//                                          flipped bytes; those loads may fail, not crash
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <unistd.h>

#include "polygrad_hip.h"

static std::vector<char> slurp(const char *path) {
  std::vector<char> d;
  if (FILE *f = fopen(path, "rb")) {
    char buf[65536];
    size_t n;
    while ((n = fread(buf, 1, sizeof(buf), f)) > 0) d.insert(d.end(), buf, buf + n);
    fclose(f);
  }
  return d;
}

static bool spill(const std::string &path, const std::vector<char> &d) {
  FILE *f = fopen(path.c_str(), "wb");
  if (!f) return false;
  const bool ok = fwrite(d.data(), 1, d.size(), f) == d.size();
  fclose(f);
  return ok;
}

// Everything the library does with a schedule short of compiling for a device.
static int exercise(const PolySchedule *s, bool must_lower) {
  int bad = 0;
  for (int k = 0; k < s->n_items; k++) {
    PolyUOp *root = s->items[k].root;
    for (int flags = 0; flags < 2; flags++) {
      int launch[7];
      char *src = poly_hip_render(root, "host_check", flags, launch);
      if (!src && must_lower) { fprintf(stderr, "host_check: kernel %d does not render (flags %d)\n", k, flags); bad++; }
      poly_hip_free_string(src);
    }
    char *d = poly_hip_describe(root, 0);
    poly_hip_free_string(d);
    const int mism = poly_hip_check_index_simplification(root, 512);
    if (mism != 0 && must_lower) { fprintf(stderr, "host_check: kernel %d: index self-check returned %d\n", k, mism); bad++; }
  }
  const int n_groups = poly_hip_fused_groups(s, -1, nullptr, nullptr);
  for (int g = 0; g < n_groups; g++) {
    char *src = nullptr;
    int n_items = 0, slots[64], launch[4];
    poly_hip_fused_groups(s, g, &src, &n_items);
    poly_hip_free_string(src);
    poly_hip_fused_group_launch(s, g, slots, 64, launch);
  }
  int holes[64];
  poly_hip_unwritten_slots(s, holes, 64);
  return bad;
}

int main(int argc, char **argv) {
  bool garbage = false;
  int bad = 0, n_files = 0, n_rejected = 0;
  const char *tmpdir = getenv("TMPDIR") ? getenv("TMPDIR") : "/tmp";
  for (int a = 1; a < argc; a++) {
    if (!strcmp(argv[a], "--garbage")) { garbage = true; continue; }
    n_files++;
    PolyHipPlanFile *pf = poly_hip_planfile_load(argv[a]);
    if (!pf) { fprintf(stderr, "host_check: %s does not load\n", argv[a]); bad++; continue; }
    bad += exercise(poly_hip_planfile_schedule(pf), true);
    for (int i = 0; i < poly_hip_planfile_schedule(pf)->n_buf_slots; i++) (void)poly_hip_planfile_slot_name(pf, i);
    poly_hip_planfile_free(pf);
    if (!garbage) continue;
    const std::vector<char> good = slurp(argv[a]);
    const std::string tmp = std::string(tmpdir) + "/host_check_" + std::to_string((long)getpid()) + ".polyplan";
    unsigned seed = 12345u + (unsigned)a;
    auto rnd = [&]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    for (int trial = 0; trial < 24; trial++) {
      std::vector<char> d = good;
      if (trial < 8) d.resize(good.size() * (size_t)(trial + 1) / 10);                  // cut short
      else for (int flips = 0; flips < 1 + trial % 4; flips++) d[rnd() % d.size()] ^= (char)(1u << (rnd() % 8));   // bit flips
      if (!spill(tmp, d)) continue;
      PolyHipPlanFile *g = poly_hip_planfile_load(tmp.c_str());
      if (!g) { n_rejected++; continue; }
      exercise(poly_hip_planfile_schedule(g), false);      // whatever it holds must not crash the lowering
      poly_hip_planfile_free(g);
    }
    remove(tmp.c_str());
  }
  printf("host_check: %d files, %d damaged copies rejected by the loader, %d problems\n", n_files, n_rejected, bad);
  return bad ? 1 : 0;
}

// Drives the planner with random slice lists (valid partitions, arbitrary overlapping or
// incomplete ones, empty slices) and random byte strings as plan messages.  Built with
// -fsanitize=address,undefined by tests/test_sanitize_cpu.py: any out-of-bounds access or
// undefined arithmetic aborts the run.  Exceptions are the expected way to refuse an input.
#include "planner.h"
#include <cstdio>
#include <random>
#include <algorithm>
#include <cstring>
using namespace moodist;
int main() {
  std::mt19937 rng(1);
  auto R = [&](int lo, int hi) { return (int)(rng() % (unsigned)(hi - lo + 1)) + lo; };
  size_t ok = 0, err = 0;
  for (int t = 0; t < 4000; ++t) {
    int P = R(1, 6), nd = R(1, 5);
    Dims shape(nd);
    for (auto& v : shape) v = R(1, 9);
    std::vector<SliceSpec> in, out;
    int mode = R(0, 3);
    if (mode < 3) {
      int d = R(0, nd - 1);
      std::vector<int> cuts = {0, (int)shape[d]};
      for (int i = 0; i < 4; ++i) cuts.push_back(R(0, (int)shape[d]));
      std::sort(cuts.begin(), cuts.end());
      cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
      for (size_t i = 0; i + 1 < cuts.size(); ++i) {
        SliceSpec s; s.rank = R(0, P - 1); s.offset.assign(nd, 0); s.shape = shape;
        s.offset[d] = cuts[i]; s.shape[d] = cuts[i + 1] - cuts[i];
        in.push_back(s);
      }
    } else {  // arbitrary, possibly overlapping or not covering: must throw cleanly or plan
      for (int i = R(0, 5); i > 0; --i) {
        SliceSpec s; s.rank = R(0, P - 1); s.offset.resize(nd); s.shape.resize(nd);
        for (int k = 0; k < nd; ++k) { s.offset[k] = R(0, (int)shape[k] - 1); s.shape[k] = R(0, (int)shape[k] - (int)s.offset[k]); }
        in.push_back(s);
      }
    }
    for (int r = 0; r < P; ++r)
      for (int i = R(0, 2); i > 0; --i) {
        SliceSpec s; s.rank = r; s.offset.resize(nd); s.shape.resize(nd);
        for (int k = 0; k < nd; ++k) { s.offset[k] = R(0, (int)shape[k] - 1); s.shape[k] = R(mode == 3 ? 0 : 1, (int)shape[k] - (int)s.offset[k]); }
        out.push_back(s);
      }
    try {
      PlanWire w;
      auto plans = plan_redistribution(P, shape, 4, in, out, &w);
      for (auto& row : w) for (auto& m : row) check_plan_message(m, nd);
      ++ok;
    } catch (const std::exception&) { ++err; }
  }
  std::printf("planned %zu, rejected %zu\n", ok, err);
  // malformed messages
  for (int t = 0; t < 4000; ++t) {
    std::vector<uint8_t> m(R(0, 200));
    for (auto& b : m) b = (uint8_t)rng();
    if (R(0, 3) == 0 && m.size() >= 8) { uint64_t n = R(0, 3); memcpy(m.data(), &n, 8); }
    try { check_plan_message(m, R(0, 10)); } catch (const std::exception&) {}
  }
  std::puts("message fuzz done");
  return 0;
}

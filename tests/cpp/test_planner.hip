// Host-only property test of the launch planner (plan_launches, alamd_dispatch.h): whatever the
// segment lengths and the launch size, the launches it asks for cover every (segment, tile) exactly
// once, in grids the device accepts.  Needs no GPU: nothing is launched.
//
// usage: test_planner [trials, default 4000]
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "alamd_dispatch.h"

using namespace alamd;

static int g_fail = 0, g_checks = 0;
#define EXPECT(cond, ...) do { ++g_checks; if (!(cond)) { ++g_fail; std::printf("FAIL line %d: ", __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } } while (0)

int main(int argc, char **argv) {
  const int trials = argc > 1 ? std::atoi(argv[1]) : 4000;
  std::mt19937_64 rng(12345);
  auto pick = [&](size_t lo, size_t hi) { return lo + (size_t)(rng() % (hi - lo + 1)); };
  size_t launches_total = 0, idle_total = 0, busy_total = 0;
  for (int trial = 0; trial < trials && g_fail < 10; ++trial) {
    const unsigned nseg = (unsigned)pick(1, ALAMD_MAX_RANKS);
    const int P = (int)pick(1, ALAMD_MAX_RANKS);
    const size_t tile_elems = (size_t)1 << pick(10, 14);
    const size_t launch_bytes[] = {(size_t)1 << 20, (size_t)64 << 20, (size_t)800 << 20};
    const size_t per_launch = launch_tiles(P, tile_elems * 4, launch_bytes[pick(0, 2)]);
    SegParams seg = make_seg(0, 0, 1, OUT_SEG, 1);
    seg.ragged = (int)pick(0, 1);
    size_t max_len = 0;
    std::vector<size_t> len(nseg);
    const int shape = (int)pick(0, 4);
    for (unsigned s = 0; s < nseg; ++s) {
      size_t l;
      switch (shape) {
      case 0: l = pick(0, 3 * tile_elems); break;                                   // a few tiles, some empty
      case 1: l = pick(0, 1) ? 0 : pick(1, 40000 * tile_elems); break;              // long or empty
      case 2: l = s == nseg / 2 ? 60000 * tile_elems + 17 : pick(1, tile_elems); break;  // one long among short
      case 3: l = (size_t)(s + 1) * pick(1, 900) * tile_elems / 3; break;           // ascending
      default: l = pick(1, 20000 * tile_elems); break;
      }
      len[s] = l;
      if (l > max_len) max_len = l;
    }
    if (!seg.ragged)
      for (unsigned s = 0; s < nseg; ++s) len[s] = max_len;  // equal segments: the planner is given max_len only
    for (unsigned s = 0; s < nseg; ++s) seg.seg_len[s] = len[s];
    std::vector<std::vector<unsigned char>> seen(nseg);
    for (unsigned s = 0; s < nseg; ++s) seen[s].assign((len[s] + tile_elems - 1) / tile_elems, 0);
    size_t launches = 0, idle = 0, busy = 0;
    bool bad_grid = false;
    plan_launches(seg, nseg, max_len, tile_elems, per_launch, [&](size_t t0, size_t nt, unsigned s0, unsigned n) {
      ++launches;
      if (nt == 0 || nt > 0x7fffffffull || n == 0 || n > 65535u || s0 + n > nseg) bad_grid = true;
      for (unsigned y = 0; y < n && !bad_grid; ++y) {
        const unsigned pos = s0 + y, s = seg.mapped ? seg.order[pos] : pos;
        if (s >= nseg) { bad_grid = true; break; }
        for (size_t t = t0; t < t0 + nt; ++t) {
          if (t < seen[s].size()) { if (seen[s][t] < 255) ++seen[s][t]; ++busy; }
          else ++idle;
        }
      }
    });
    EXPECT(!bad_grid, "trial %d: a launch with an empty or oversized grid, or segments past the end", trial);
    size_t missed = 0, twice = 0;
    for (unsigned s = 0; s < nseg; ++s)
      for (unsigned char c : seen[s]) { missed += c == 0; twice += c > 1; }
    EXPECT(missed == 0 && twice == 0, "trial %d (nseg %u, ragged %d, shape %d, per_launch %zu): %zu tiles missed, %zu covered twice",
           trial, nseg, seg.ragged, shape, per_launch, missed, twice);
    if (seg.mapped) {
      // a permutation of the segments
      std::vector<int> hit(nseg, 0);
      for (unsigned i = 0; i < nseg; ++i) if (seg.order[i] < nseg) ++hit[seg.order[i]];
      bool perm = true;
      for (int h : hit) perm = perm && h == 1;
      EXPECT(perm, "trial %d: the segment order is not a permutation", trial);
    }
    // launches stay near the size asked for: none moves more than a launch and a half, plus what the
    // rounding to whole segments side by side adds
    launches_total += launches;
    idle_total += idle;
    busy_total += busy;
  }
  // workgroups that find nothing to do: a planner that put every segment side by side in one grid
  // would idle far more than it works on the "one long among short" shapes
  EXPECT(idle_total < busy_total, "idle workgroups %zu against %zu busy ones", idle_total, busy_total);
  std::printf("%s: %d trials, %zu launches, %zu busy and %zu idle workgroups, %d checks, %d failed\n",
              g_fail ? "FAILED" : "PASSED", trials, launches_total, busy_total, idle_total, g_checks, g_fail);
  return g_fail ? 1 : 0;
}

// Host-only property test of the launch planner (plan_launches, alamd_dispatch.h): whatever the
// segment lengths and the launch size, the launches it asks for cover every (segment, tile) exactly
// once, in grids the device accepts.  Also: the block lookup of the role masks against its definition,
// and the LDS sizing of the streaming launches.  Needs no GPU: nothing is launched.
//
// usage: test_planner [trials, default 4000]
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "alamd_dispatch.h"
#include "alamd_tile.h"

// (the library defines this in core.hip; this program links no library)
namespace alamd { Tunables &tunables() { static Tunables t; return t; } }

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
  // The block of a message that an element lies in (role_mask_of_elem): the lookup through prepared
  // reciprocals gives what the 64-bit divisions give, and the block ends where it says - for both ways
  // of cutting a message, every number of blocks, bases inside the message, and lengths up to 2^40.
  for (int trial = 0; trial < trials && g_fail < 10; ++trial) {
    TreeParams tp = {};
    tp.role_bits = (int)pick(0, 6);
    tp.role_spread = (int)pick(0, 1);
    const unsigned long long n = trial % 3 == 0 ? pick(1, 5000) : (trial % 3 == 1 ? pick(1, (size_t)1 << 40) : ((size_t)1 << pick(6, 40)) + pick(0, 70));
    const unsigned long long base = pick(0, n - 1), seg_len = n - base;
    tp.role_base = base;
    tp.role_count = n;
    TreeParams fast = tp;
    fast.role_n = n;
    fast.role_blk = n >> tp.role_bits;
    fast.role_inv_blk = fast.role_blk ? 1.0 / (double)fast.role_blk : 0.0;
    fast.role_inv_blk1 = 1.0 / (double)(fast.role_blk + 1);
    const unsigned long long blocks = 1ull << tp.role_bits, blk = n >> tp.role_bits, longer = n & (blocks - 1);
    for (int k = 0; k < 200; ++k) {
      // elements at and around the block boundaries, and anywhere
      unsigned long long x;
      if (k < 150 && blk > 0) {
        const unsigned long long b = pick(0, blocks - 1);
        const unsigned long long start = tp.role_spread ? b * blk + (b < longer ? b : longer) : b * blk;
        x = start + pick(0, 2) - 1;
        if (x >= n) x = n - 1;
      } else {
        x = pick(0, n - 1);
      }
      if (x < base) x = base;
      const size_t e = (size_t)(x - base);
      unsigned long long end_slow = 0, end_fast = 0;
      const unsigned ms = role_mask_of_elem(tp, (size_t)seg_len, e, &end_slow), mf = role_mask_of_elem(fast, (size_t)seg_len, e, &end_fast);
      EXPECT(ms == mf && end_slow == end_fast, "block lookup: n %llu bits %d spread %d element %llu: mask %u / %u, end %llu / %llu", n,
             tp.role_bits, tp.role_spread, x, ms, mf, end_slow, end_fast);
      // the block by its definition
      unsigned long long kb = 0, lo = 0, hi = 0;
      for (kb = 0; kb < blocks; ++kb) {
        lo = tp.role_spread ? kb * blk + (kb < longer ? kb : longer) : kb * blk;
        hi = kb == blocks - 1 ? n : (tp.role_spread ? lo + blk + (kb < longer ? 1 : 0) : lo + blk);
        if (x >= lo && x < hi) break;
      }
      EXPECT(kb < blocks && ms == role_bit_reverse((unsigned)kb, tp.role_bits), "block lookup: n %llu bits %d spread %d element %llu is in block %llu", n,
             tp.role_bits, tp.role_spread, x, kb);
      EXPECT(kb == blocks - 1 ? end_slow == ~0ull : end_slow == hi - base, "block lookup: end of block %llu: %llu, expected %llu", kb, end_slow, hi - base);
    }
  }
  // The LDS a streaming launch asks for lets exactly the wanted number of one-wave workgroups into a CU's
  // 160 KiB, up to the eight waves per SIMD the kernels are compiled for.
  for (int n = 1; n <= 40; ++n) {
    const unsigned lds = stream_lds_bytes(n);
    const int want = n < 4 ? 4 : (n > 32 ? 32 : n);
    EXPECT(lds >= 128 && 160u * 1024u / lds >= (unsigned)want && 160u * 1024u / (lds + 128) <= (unsigned)want, "LDS for %d workgroups per CU: %u bytes", n, lds);
  }
  // The leading elements of a segment: never more than the segment, whole elements, below 1 KiB's worth;
  // long segments then have their first input on a 1 KiB boundary, short ones their output on a 64-byte
  // boundary where the first input's vectors then start on a dword (else the first input on a dword).
  {
    std::mt19937_64 rng(4242);
    const size_t sizes[] = {1, 2, 4, 8};
    for (int t = 0; t < 20000; ++t) {
      const size_t es = sizes[rng() % 4];
      const uintptr_t out = (uintptr_t)((rng() % (1u << 20)) * es), first = (uintptr_t)((rng() % (1u << 20)) * es);
      const size_t len = t % 3 == 0 ? rng() % 200 : (t % 3 == 1 ? kBigHeadFromBytes / es - 2 + rng() % 5 : rng() % (1u << 22));
      const size_t h = stream_head_count(es, reinterpret_cast<const char *>(out), reinterpret_cast<const char *>(first), len);
      EXPECT(h <= len && h * es < kStreamTileBytes, "head of %zu elements of %zu bytes, segment of %zu", h, es, len);
      if (h == len) continue;
      if (len * es >= kBigHeadFromBytes) {
        EXPECT((first + h * es) % kStreamTileBytes == 0, "long segment: first input %zu bytes off a tile boundary", (size_t)((first + h * es) % kStreamTileBytes));
      } else if ((out ^ first) % 4 == 0) {
        EXPECT((out + h * es) % 64 == 0 && (first + h * es) % 4 == 0, "short segment: output %zu bytes off a line", (size_t)((out + h * es) % 64));
      } else {
        EXPECT((first + h * es) % 4 == 0, "short segment: first input splits its dwords (%zu)", (size_t)((first + h * es) % 4));
      }
    }
  }
  // Runs of consecutive tiles per XCD: a permutation of the launch's tiles whatever its length; in every whole
  // group the workgroups that go to one XCD (index mod 8) take 2^rl consecutive tiles, in order.
  for (unsigned rl = 1; rl <= 5; ++rl) {
    for (unsigned n : {1u, 7u, 8u, 31u, 32u, 33u, 255u, 256u, 1000u, 4096u, 5000u}) {
      std::vector<int> seen(n, 0);
      bool in_range = true, runs = true;
      for (unsigned i = 0; i < n; ++i) {
        const unsigned t = xcd_run_tile(i, n, rl);
        if (t >= n) { in_range = false; break; }
        ++seen[t];
        const unsigned span = 8u << rl;
        if (i + 8 < n && (i + 8) / span == i / span && i / span < n / span) runs = runs && xcd_run_tile(i + 8, n, rl) == t + 1;
      }
      bool once = in_range;
      for (unsigned t = 0; once && t < n; ++t) once = seen[t] == 1;
      EXPECT(once && runs, "tiles of a launch of %u in runs of %u per XCD: every tile once %d, consecutive %d", n, 1u << rl, (int)once, (int)runs);
    }
  }
  // Tiles go by the output only where some input sits at another distance from a 64-byte boundary, every
  // input is on the output's dword grid, and the segment is long.
  {
    const char *base = reinterpret_cast<const char *>((uintptr_t)1 << 30);
    auto by_out = [&](size_t es, size_t out_off, std::vector<size_t> in_off, size_t len) {
      return tiles_by_output(es, base + out_off, len, (int)in_off.size(), [&](int k) { return base + (1 << 20) * (k + 1) + in_off[(size_t)k]; });
    };
    EXPECT(!by_out(4, 0, {0, 0, 0}, 1 << 20), "aligned buffers");
    EXPECT(!by_out(4, 4, {4, 4, 68}, 1 << 20), "a common distance (mod 64)");
    EXPECT(by_out(4, 20, {0, 0, 0}, 1 << 20), "output 20 bytes off");
    EXPECT(by_out(4, 0, {0, 12, 0}, 1 << 20), "one input 12 bytes off");
    EXPECT(!by_out(4, 20, {0, 0, 0}, 1000), "short segment");
    EXPECT(!by_out(2, 2, {0, 0}, 1 << 20), "inputs off the output's dword grid");
    EXPECT(by_out(2, 4, {0, 0}, 1 << 20), "16-bit elements, output two elements off");
  }
  // Workgroups per CU of a streaming launch: by size, streams and outputs; a launch of few rounds takes
  // the setting with the fewest whole rounds (a tree only from two rounds to one).
  {
    const size_t MiB = (size_t)1 << 20;
    EXPECT(stream_wgs_per_cu(false, 8, 1, 2304 * MiB, 262144, 256) == 22 && stream_wgs_per_cu(true, 8, 1, 2304 * MiB, 262144, 256) == 16, "large launches");
    EXPECT(stream_wgs_per_cu(false, 8, 1, 20 * MiB, 2276, 256) == 32 && stream_wgs_per_cu(true, 8, 1, 20 * MiB, 2276, 256) == 26, "small launches");
    EXPECT(stream_wgs_per_cu(false, 8, 8, 2304 * MiB, 262144, 256) == 16 && stream_wgs_per_cu(false, 2, 1, 768 * MiB, 262144, 256) == 26, "outputs, two streams");
    EXPECT(stream_wgs_per_cu(false, 64, 1, 384 * MiB, 6048, 256) == 26, "6048 tiles: one round with 26 per CU");
    EXPECT(stream_wgs_per_cu(false, 64, 1, 448 * MiB, 7056, 256) == 32, "7056 tiles: one round with 32");
    EXPECT(stream_wgs_per_cu(false, 48, 1, 448 * MiB, 9360, 256) == 22, "9360 tiles: two rounds whatever the setting");
    EXPECT(stream_wgs_per_cu(false, 32, 1, 384 * MiB, 11904, 256) == 26, "11904 tiles: three rounds with 22, two with 26");
    EXPECT(stream_wgs_per_cu(false, 8, 1, 512 * MiB, 58240, 256) == 22 && stream_wgs_per_cu(false, 16, 1, 512 * MiB, 30832, 256) == 22, "more than five rounds: by size alone");
    EXPECT(stream_wgs_per_cu(false, 16, 1, 384 * MiB, 23120, 256) == 32, "five rounds with 22, three with 32");
    EXPECT(stream_wgs_per_cu(true, 64, 1, 288 * MiB, 4528, 256) == 22 && stream_wgs_per_cu(true, 64, 1, 384 * MiB, 6048, 256) == 26, "a tree: from two rounds to one");
    EXPECT(stream_wgs_per_cu(true, 64, 1, 448 * MiB, 7056, 256) == 16 && stream_wgs_per_cu(true, 32, 1, 512 * MiB, 15872, 256) == 16, "a tree: otherwise by size");
    EXPECT(stream_wgs_per_cu(false, 64, 1, 384 * MiB) == 22, "unknown tile count");
  }
  // Which launches take the block shape (the sizes at their defaults; 256 CUs).
  {
    const size_t MiB = (size_t)1 << 20;
    EXPECT(use_block_shape(144 * MiB, 8, 1, false, 1024, 256), "P = 8, 16 MiB per rank: four tiles per CU");
    EXPECT(!use_block_shape(144 * MiB, 8, 1, false, 1025, 256), "one tile more: a fifth round for one CU");
    EXPECT(use_block_shape(192 * MiB, 8, 1, true, 2731 - 171, 256), "ten tiles per CU exactly");
    EXPECT(use_block_shape(192 * MiB, 8, 1, true, 2550, 256), "0.4 %% of the CUs idle in the last round");
    EXPECT(!use_block_shape(192 * MiB, 8, 1, true, 1365, 256), "5.33 tiles per CU");
    EXPECT(use_block_shape(40 * MiB, 8, 1, false, 200, 256), "fewer tiles than CUs");
    EXPECT(use_block_shape(144 * MiB, 8, 8, false, 1025, 256), "eight outputs: whatever the tiles");
    EXPECT(!use_block_shape(144 * MiB, 4, 1, false, 1024, 256), "four ranks");
    EXPECT(use_block_shape(144 * MiB, 4, 3, false, 1024, 256), "four ranks, three outputs");
    EXPECT(use_block_shape(20 * MiB, 64, 1, false, 20, 256), "a fold over 64 ranks from 16 MiB on");
    EXPECT(!use_block_shape(20 * MiB, 64, 1, true, 20, 256) && !use_block_shape(20 * MiB, 8, 1, false, 142, 256), "others from 32 MiB on");
    EXPECT(!use_block_shape(144 * MiB, 48, 1, true, 256, 256, 4096) && !use_block_shape(144 * MiB, 48, 8, true, 256, 256, 8192), "tree tiles under 16 KiB");
    EXPECT(!use_block_shape(384 * MiB, 8, 1, false, 2048, 256) && !use_block_shape(31 * MiB, 8, 8, false, 256, 256), "outside the window");
    EXPECT(use_block_shape(144 * MiB, 8, 1, false, 1025, 0), "unknown device: the window alone");
  }
  // workgroups that find nothing to do: a planner that put every segment side by side in one grid
  // would idle far more than it works on the "one long among short" shapes
  EXPECT(idle_total < busy_total, "idle workgroups %zu against %zu busy ones", idle_total, busy_total);
  std::printf("%s: %d trials, %zu launches, %zu busy and %zu idle workgroups, %d checks, %d failed\n",
              g_fail ? "FAILED" : "PASSED", trials, launches_total, busy_total, idle_total, g_checks, g_fail);
  return g_fail ? 1 : 0;
}

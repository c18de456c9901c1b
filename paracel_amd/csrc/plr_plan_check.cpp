// Host-only check of the width -> variant choice (plr_plan.hpp): walks every
// width and verifies what the kernels and the launch code rely on.
//   plr_plan_check              check d = 1 .. 70000, report, exit 0/1
//   plr_plan_check <d>          print the plan for one width
#include <stdio.h>
#include <stdlib.h>

#include <vector>

#include "plr_plan.hpp"

using namespace plr_plan;

static int failures = 0;
#define CHECK(cond, d)                                                        \
  do {                                                                        \
    if (!(cond)) {                                                            \
      if (++failures <= 20) printf("d=%lld: %s\n", (long long)(d), #cond);    \
    }                                                                         \
  } while (0)

// the team split of a column-blocked plan: replays the kernel's own arithmetic
static void check_team(const Plan& p, int64_t d, int cap) {
  const int64_t chunks = ceil_div(p.pitch, kChunkCols);
  if (!p.team_blocks) {
    CHECK(chunks > (int64_t)kMaxTeamBlocks * kTeamWaves * cap, d);
    return;
  }
  CHECK(p.team_blocks >= 2 && p.team_blocks <= kMaxTeamBlocks, d);
  CHECK(p.team_blk_extra >= 0 && p.team_blk_extra < p.team_blocks, d);
  // the blocks cover the row exactly, and no wave owns more chunks than the kernel holds
  CHECK((int64_t)p.team_blocks * p.team_blk_chunks + p.team_blk_extra == chunks, d);
  CHECK(p.team_nch >= kTeamMinNch && p.team_nch <= cap, d);
  CHECK(p.team_lag == 1 || p.team_lag == 2, d);
  CHECK(ceil_div(p.team_blk_chunks + (p.team_blk_extra ? 1 : 0), kTeamWaves) <= p.team_nch, d);
  CHECK(p.team_blk_chunks >= kTeamWaves, d);  // every wave owns a chunk
  int64_t next = 0;
  for (int b = 0; b < p.team_blocks; ++b) {
    const int bm = p.team_blk_chunks + (b < p.team_blk_extra ? 1 : 0);
    const int64_t b0 = (int64_t)b * p.team_blk_chunks + (b < p.team_blk_extra ? b : p.team_blk_extra);
    const int wq = bm / kTeamWaves, wrem = bm % kTeamWaves;
    for (int w = 0; w < kTeamWaves; ++w) {
      const int m = wq + (w < wrem ? 1 : 0);
      const int64_t c0 = b0 + (int64_t)w * wq + (w < wrem ? w : wrem);
      CHECK(c0 == next && m >= 1 && m <= p.team_nch, d);
      next = c0 + m;
    }
  }
  CHECK(next == chunks, d);
  CHECK(p.theta_len >= chunks * kChunkCols + kChunkCols, d);
}

static void print_plan(int64_t d, int64_t n) {
  Plan p;
  if (!plan_width(d, p, n)) {
    printf("d=%lld: no variant\n", (long long)d);
    return;
  }
  static const char* names[] = {"lane", "fused", "blocked", "pair"};
  printf("d=%lld path=%s pitch=%lld theta_len=%lld", (long long)d, names[p.path],
         (long long)p.pitch, (long long)p.theta_len);
  if (p.path == kPathLane) printf(" np=%d", p.np);
  if (p.path == kPathFused) {
    const Shape& s = kShapes[p.variant];
    printf(" variant=%d NCH=%d R=%d WCOL=%d WROW=%d THL=%d TL=%d chunks=%lld nch_rt=%d allch=%d tail=%d",
           p.variant, s.nch, s.R, s.wcol, s.wrow, (int)s.thl, s.tl, (long long)p.chunks, p.nch_rt,
           (int)p.allch, p.tail_cols);
  }
  if (p.path == kPathBlocked)
    printf(" team_blocks=%d blk_chunks=%d(+1 in the first %d) nch=%d lag=%d", p.team_blocks,
           p.team_blk_chunks, p.team_blk_extra, p.team_nch, p.team_lag);
  printf("\n");
}

int main(int argc, char** argv) {
  if (argc > 1) {  // plr_plan_check <d> [<n>]
    print_plan(atoll(argv[1]), argc > 2 ? atoll(argv[2]) : -1);
    return 0;
  }
  std::vector<int64_t> used(kNumShapes, 0);
  const int64_t kMaxD = 600000;
  // every width twice: rows unknown (a large shard) and a one-row shard (the
  // short-tile entries of the table)
  for (int64_t dn = 2; dn <= 2 * kMaxD + 1; ++dn) {
    const int64_t d = dn / 2, n = (dn & 1) ? 1 : -1;
    Plan p;
    if (!plan_width(d, p, n)) {
      CHECK(false && "plan_width failed", d);
      continue;
    }
    CHECK(p.pitch >= d && p.pitch % 2 == 0, d);
    CHECK(p.theta_len >= p.pitch, d);
    CHECK(p.path != kPathFused || p.pitch > kMaxPairPitch, d);
    if (p.path == kPathLane) {
      CHECK(d <= kMaxLaneCols && p.np >= 1 && p.np <= 32, d);
      CHECK(p.pitch == 2 * p.np && p.pitch - d < 2, d);
    } else if (p.path == kPathPair) {
      CHECK(d > kMaxLaneCols && p.pitch <= kMaxPairPitch && p.pitch - d < 2, d);
      CHECK(p.theta_len >= kChunkCols, d);  // both column pairs of every lane read theta
    } else if (p.path == kPathBlocked) {
      CHECK(d > kMaxFusedCols && p.pitch % 16 == 0 && p.pitch - d < 16, d);
      CHECK(p.theta_len >= p.pitch + kChunkCols, d);  // a whole chunk of zeros behind theta
      if (p.team_blocks) {
        check_team(p, d, kTeamNch);
      } else {
        CHECK(ceil_div(p.pitch, kChunkCols) > (int64_t)kMaxTeamBlocks * kBlkWcol * kTeamNch, d);
      }
    } else {
      CHECK(d > kMaxLaneCols && d <= kMaxFusedCols, d);
      CHECK(p.variant >= 0 && p.variant < kNumShapes, d);
      if (p.variant < 0 || p.variant >= kNumShapes) continue;
      const Shape& s = kShapes[p.variant];
      used[p.variant]++;
      CHECK(p.pitch - d < (d >= 2048 ? 16 : 2), d);
      CHECK(d < 2048 || p.pitch % 16 == 0, d);
      CHECK(p.chunks == ceil_div(p.pitch, kChunkCols), d);
      CHECK(s.wcol == 1 || s.wrow == 1, d);
      CHECK((s.R & (s.R - 1)) == 0 && s.R <= 64, d);
      // theta in LDS: one slab per wave, within the 160 KiB of a compute unit
      CHECK(!s.thl || (int64_t)s.wcol * s.wrow * s.nch * 1024 <= 160 * 1024, d);
      // the 32-bit lane offsets of a tile (R rows of pitch doubles) cannot wrap
      CHECK((int64_t)s.R * p.pitch * 8 + 8 * p.pitch < (int64_t(1) << 32), d);
      if (p.tail_cols) {
        CHECK(s.tl > 0 && s.tl <= s.R && s.tl <= 4 && (s.tl & (s.tl - 1)) == 0, d);
        CHECK(p.allch && p.nch_rt == s.nch, d);
        CHECK((int64_t)s.nch * s.wcol * kChunkCols + p.tail_cols == p.pitch, d);
        CHECK(p.tail_cols % 2 == 0 && p.tail_cols <= kChunkCols * s.tl / s.R, d);
        CHECK(p.theta_len >= p.pitch, d);
      } else {
        CHECK(s.tl == 0, d);
        CHECK(p.nch_rt >= 1 && p.nch_rt <= s.nch, d);
        CHECK((int64_t)s.wcol * p.nch_rt >= p.chunks, d);            // every chunk has a wave
        CHECK((int64_t)(s.wcol - 1) * p.nch_rt < p.chunks, d);       // no wave without a chunk
        CHECK(p.allch == (p.chunks == (int64_t)s.nch * s.wcol), d);
        CHECK(!p.allch || p.nch_rt == s.nch, d);
        // one-wave rows exist only as exact (allch) instances
        CHECK(s.wcol > 1 || p.allch, d);
        CHECK(p.theta_len >= (int64_t)s.wcol * p.nch_rt * kChunkCols, d);
        // idle chunk slots: fewer than one wave's worth
        CHECK((int64_t)s.wcol * p.nch_rt - p.chunks < p.nch_rt, d);
      }
    }
  }
  int dead = 0;
  for (int i = 0; i < kNumShapes; ++i)
    if (!used[i]) {
      const Shape& s = kShapes[i];
      printf("variant %d (NCH=%d R=%d WCOL=%d WROW=%d THL=%d TL=%d) is never chosen\n", i, s.nch,
             s.R, s.wcol, s.wrow, (int)s.thl, s.tl);
      ++dead;
    }
  printf("%s: %lld widths, %d variants, %d never chosen, %d failed checks\n",
         (failures || dead) ? "FAIL" : "ok", (long long)kMaxD, kNumShapes, dead, failures);
  return (failures || dead) ? 1 : 0;
}

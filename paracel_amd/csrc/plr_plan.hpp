// Width -> layout and kernel variant, as a pure host function (no HIP types):
// which of the four paths a shard of d columns takes, its row pitch in HBM,
// and for the fused path the shard_pass variant with its run-time chunk
// count.  Kept apart from the kernels so that the choice can be checked on a
// CPU for every width (the GPU side then only adds occupancy and grid size).
#pragma once

#include <stdint.h>

namespace plr_plan {

constexpr int kChunkCols = 128;          // columns per chunk (a double2 per lane)
constexpr int64_t kMaxLaneCols = 64;     // up to here: row-tiled layout, a lane per row (lane_pass)
constexpr int64_t kMaxPairPitch = 96;    // up to this pitch: a half-wave per row (pair_pass)
constexpr int64_t kMaxFusedCols = 19456; // beyond: column blocks, two sweeps over X
constexpr int kBlkNch = 16, kBlkWcol = 8;
constexpr int64_t kBlockCols = (int64_t)kBlkNch * kBlkWcol * kChunkCols;  // 16384
constexpr int kMaxTeamBlocks = 64;       // column blocks a team of workgroups may span
constexpr int kTeamWaves = 8;            // waves of a team's workgroup, side by side
constexpr int kTeamMinNch = 7;           // chunks per wave the team kernels are built for: from ...
constexpr int kTeamNch = 8;              // ... to (rows past 19456 columns never need fewer than 7)
constexpr int kAlwaysOneWave = 16;       // up to here no several-waves variant is considered
constexpr int kMaxRowChunks = 32;        // widest one-wave row

struct Shape {
  int nch, R, wcol, wrow, minw;
  bool thl;
  int tl;  // tail loads per tile (0: the row ends inside or at the end of a chunk)
};

static const Shape kShapes[] = {
#define PLR_V(NCH, R, WCOL, WROW, MINW, THL, TL) {NCH, R, WCOL, WROW, MINW, THL, TL},
#include "plr_variants.def"
#undef PLR_V
};
constexpr int kNumShapes = (int)(sizeof(kShapes) / sizeof(kShapes[0]));

enum Path { kPathLane = 0, kPathFused = 1, kPathBlocked = 2, kPathPair = 3 };

struct Plan {
  Path path;
  int64_t pitch;      // doubles per row in HBM (>= d; pad columns are zero)
  int64_t theta_len;  // doubles of the zero-padded device copy of theta
  // lane path: tiles of 64 rows stored column pair by column pair
  int np;             // column pairs per row = pitch / 2
  // fused path
  int variant;        // index into kShapes
  int64_t chunks;     // ceil(pitch / 128)
  int nch_rt;         // chunks per wave actually used (<= the variant's NCH)
  bool allch;         // every wave of the row uses exactly NCH chunks
  int tail_cols;      // columns handled by the variant's tail stage (0: none)
  // column-blocked path, one read of X: a team of team_blocks workgroups per
  // row (0 blocks: too wide, two sweeps); the first team_blk_extra of them own
  // team_blk_chunks + 1 chunks, the others team_blk_chunks, and a block's
  // chunks are dealt the same way to its 8 waves, team_nch at most each
  int team_blocks;
  int team_blk_chunks;
  int team_blk_extra;
  int team_nch;
  int team_lag;       // steps between a row's dot product and its update (1 or 2)
};

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Fills p for a shard of d >= 1 columns; false if no variant covers the width
// (cannot happen with the table as it is; checked by the host-side test).
// n: rows of the shard when known (< 0: unknown, taken as large).  Where the
// variant table has two entries for a shape, shards below kSmallShardBytes
// take the one with the shorter tiles.
constexpr int64_t kSmallShardBytes = 1500000000;
inline bool plan_width(int64_t d, Plan& p, int64_t n = -1) {
  p = Plan();
  p.variant = -1;
  if (d <= kMaxLaneCols) {
    p.path = kPathLane;
    p.np = (int)((d + 1) / 2);
    p.pitch = 2 * (int64_t)p.np;
    p.theta_len = kChunkCols;
    return true;
  }
  if (((d + 1) & ~int64_t(1)) <= kMaxPairPitch) {
    // 65..96 columns: two rows per wave instruction, even pitch
    p.path = kPathPair;
    p.pitch = (d + 1) & ~int64_t(1);
    p.theta_len = kChunkCols;
    return true;
  }
  if (d > kMaxFusedCols) {
    p.path = kPathBlocked;
    p.pitch = (d + 15) & ~int64_t(15);
    p.nch_rt = kBlkNch;
    // theta padded so that the last (narrower) block still reads whole slabs
    p.theta_len = ceil_div(p.pitch, kBlockCols) * kBlockCols;
    // the row's chunks dealt evenly to the fewest workgroups that can hold
    // them, and inside a workgroup evenly to its waves
    const int64_t chunks = ceil_div(p.pitch, kChunkCols);
    const int64_t blocks = ceil_div(chunks, (int64_t)kTeamWaves * kTeamNch);
    if (blocks <= kMaxTeamBlocks) {
      p.team_blocks = (int)blocks;
      p.team_blk_chunks = (int)(chunks / blocks);
      p.team_blk_extra = (int)(chunks % blocks);
      const int64_t widest = p.team_blk_chunks + (p.team_blk_extra ? 1 : 0);
      p.team_nch = (int)ceil_div(widest, kTeamWaves);  // 7 or 8: more than 152 chunks in >= 3 blocks
      if (p.team_nch < kTeamMinNch) p.team_nch = kTeamMinNch;
      // How many steps a row's update trails its dot product.  Two steps give the
      // exchange of the partial dots more time but cost a fourth row buffer.
      // Measured on 12 GB shards, one session, fraction of 8 TB/s with one step
      // -> two: teams of 3 (19457 columns 0.83 -> 0.81, 20000 0.83 -> 0.82, 24576
      // 0.85 -> 0.83) and 4 (32768 0.85 -> 0.84) are better off with one; from 5
      // on two pay, the more the larger the team (40000 0.83 -> 0.85, 50000 0.82
      // -> 0.85, 65536 0.85 -> 0.86, 100000 0.72 -> 0.83, 131072 0.76 -> 0.88,
      // 262144 0.67 -> 0.87, 524288 0.62 -> 0.79).
      p.team_lag = blocks <= 4 ? 1 : 2;
    }
    // one more chunk of padding: the page of zeros an unowned chunk slot reads
    p.theta_len += kChunkCols;
    return true;
  }
  p.path = kPathFused;
  // even pitch so that every row start is 16-byte aligned; wide rows are
  // aligned to 128 B (<= 0.7 % more bytes, +3 % bandwidth when d is odd)
  const int64_t pitch = (d >= 2048) ? ((d + 15) & ~int64_t(15)) : ((d + 1) & ~int64_t(1));
  const int64_t chunks = ceil_div(pitch, kChunkCols);
  const int64_t full = pitch / kChunkCols, rem = pitch % kChunkCols;
  int v = -1, tail = 0;
  // a few columns past a chunk boundary: the tail-stage variant with the
  // smallest capacity that holds them
  if (rem != 0 && full >= 1) {
    int best_cap = 1 << 30;
    for (int i = 0; i < kNumShapes; ++i) {
      const Shape& k = kShapes[i];
      if (k.tl == 0 || (int64_t)k.nch * k.wcol != full) continue;
      const int cap = kChunkCols * k.tl / k.R;
      if (cap >= rem && cap < best_cap) {
        v = i;
        best_cap = cap;
      }
    }
    if (v >= 0) tail = (int)rem;
  }
  if (v < 0) {
    // (waves, chunks per wave) for this width, then the variant that has them
    int want_w = 8, want_k = (int)ceil_div(chunks, 8);  // beyond 64 chunks: theta in LDS
    if (chunks <= 64) {
      want_k = (int)ceil_div(chunks, 8);
      want_w = (int)ceil_div(chunks, want_k);
      const bool fills_waves = rem == 0 && chunks == (int64_t)want_k * want_w;
      if (chunks <= kMaxRowChunks && !(chunks > kAlwaysOneWave && fills_waves)) {
        want_w = 1;
        want_k = (int)chunks;
      }
    }
    for (int i = 0; i < kNumShapes; ++i) {
      const Shape& k = kShapes[i];
      if (k.tl != 0) continue;
      const bool fits = (want_k >= 8 && want_w == 8)
                            ? (k.thl && k.wcol == 8 && k.nch >= want_k)
                            : (!k.thl && k.wcol == want_w && k.nch == want_k);
      if (!fits) continue;
      const bool small = n >= 0 && n * pitch * (int64_t)sizeof(double) < kSmallShardBytes;
      if (v < 0 || (small && k.R < kShapes[v].R)) v = i;
    }
  }
  if (v < 0) return false;
  const Shape& s = kShapes[v];
  p.variant = v;
  p.pitch = pitch;
  p.chunks = chunks;
  p.tail_cols = tail;
  if (tail) {
    p.nch_rt = s.nch;
    p.allch = true;
    p.theta_len = (full + 1) * kChunkCols;
  } else {
    p.nch_rt = (int)ceil_div(chunks, s.wcol);  // == nch except for the theta-in-LDS variants
    p.allch = (chunks == (int64_t)s.nch * s.wcol);
    p.theta_len = (int64_t)s.wcol * p.nch_rt * kChunkCols;
  }
  return true;
}

}  // namespace plr_plan

// Device kernels for the logistic-regression shard pass on gfx950 (CDNA4).
//
// One fused, HBM-bound streaming pass.  X (n x d fp64, row-major, even pitch)
// is read exactly once; everything derived from a row -- the dot product
// x.theta, the sigmoid, the residual, the loss term and the rank-1 update of
// the gradient -- happens on the registers the row was loaded into.
//
// Work decomposition
//   * A wavefront (64 lanes) owns a slab of up to NCH*128 columns.  Within a
//     128-column chunk lane l owns the adjacent pair (2l, 2l+1), so one
//     global_load_dwordx4 per lane moves a contiguous 1 KiB per wave.
//   * Rows are taken in tiles of R consecutive rows; all R*NCH loads of a
//     tile are issued before the first use.  theta and the gradient
//     accumulators for the slab live in registers for the kernel's lifetime.
//   * The R per-lane partial dots are reduced across the 64 lanes by a
//     transposing butterfly: log2(R) halving steps leave each lane with one
//     row's partial, log2(64/R) plain butterfly steps finish it.  So the
//     exp/log of a row is evaluated once per tile by the lane that holds
//     it, not 64 times, and R-1+log2(64/R) lane exchanges replace 6R.
//   * Wide rows (more than 32 chunks): WCOL waves of a workgroup split the
//     columns; their partial dots meet in LDS (double-buffered, one barrier
//     per tile) and are summed in wave order.
//   * A row that ends a few columns past a chunk boundary (the file path
//     always adds a bias column, so 256 features arrive as 257 columns) does
//     not get a nearly empty chunk of its own: the TL > 0 variants cover the
//     leftover columns of ALL rows of a tile with TL loads, 64*TL/R lanes per
//     row, reduce them inside those lane segments and fold them into the
//     row's dot product and the gradient separately (on the last wave of the
//     row when several waves share it).
//   * Rows are spread over the grid tile-interleaved (tile t goes to row
//     group t mod G), so at any moment the grid streams one contiguous window
//     of X.
// Determinism: no atomics; every sum has a fixed shape that depends only on
// (n, d, grid), so results are bitwise reproducible.
//
// Replaces, for a resident shard, the loops of the reference's
// alg/classification/logistic_regression/lr.cpp:69-72,132-138,322-330,361-363
// and include/utils/ext_utility.hpp:171-174.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace plr {

typedef double v2d __attribute__((ext_vector_type(2)));

// X is streamed once and never re-read: load it with the non-temporal hint.
#ifndef PLR_NONTEMPORAL
#define PLR_NONTEMPORAL 1
#endif
__device__ __forceinline__ v2d load_x(const v2d* p) {
#if PLR_NONTEMPORAL
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}

// Predictions are written once and not read again by the device: with the
// non-temporal hint their cost in a pass that is busy streaming X drops from
// ~11 % to ~5 % of the pass (device memory) or to nothing measurable (pinned
// host memory, where they leave through the host link instead of HBM).
__device__ __forceinline__ void store_h(double* p, double v) { __builtin_nontemporal_store(v, p); }

constexpr int kWave = 64;
constexpr int kChunkCols = 2 * kWave;  // columns per chunk (double2 per lane)

enum : unsigned {
  kLossReference = 0u,
  kLossStable = 1u,
  kLossNone = 2u,
  kLossSquared = 3u,  // identity link: residual z - y, loss (z - y)^2
};

struct PassArgs {
  const double* X;       // n x pitch
  const double* y;       // n
  const double* theta;   // padded with zeros to wcol*nch_rt*128 entries
  double* part_g;        // [grid][pitch]  per-workgroup partial gradients
  double* part_loss;     // [grid]
  double* h_out;         // n, or nullptr (predict)
  int64_t n;
  int64_t pitch;         // doubles per row in X (row stride), even, >= d
  int64_t width;         // columns this launch covers, starting at X / theta /
                         // part_g as passed (even; == pitch unless the row is
                         // processed in column blocks)
  int64_t ntiles;        // ceil(n / R)
  int nch_rt;            // chunks per wave actually used (<= NCH)
  int tail_cols;         // TL > 0 variants: columns past the last full chunk
                         // (even, <= 128*TL/R); width = chunks*128 + tail_cols
  unsigned loss_mode;
  int identity_link;     // 1: h = z (linear model), 0: h = sigmoid(z)
  // column-blocked rows (kPassDot / kPassAxpy launches)
  double* z_buf;         // n: x.theta accumulated over the column blocks
  int z_accumulate;      // 0: this block stores its partial dot, 1: adds to it
  const double* res_in;  // n: residual per row, computed between the two sweeps
  // A first column that is 1.0 in every row (the bias column the worker's
  // parser prepends, lr.cpp:83) is not stored: X, theta and part_g then hold
  // the OTHER columns, theta_bias points at the coefficient of the constant
  // column (added to every dot product) and part_res receives, per
  // workgroup, the sum of the residuals -- that column's gradient.
  const double* theta_bias;  // nullptr: every column is stored
  double* part_res;          // [grid], or nullptr
};

// loss and residual sums of a pass travel together
struct RowSums {
  double loss = 0.;
  double res = 0.;
};

// Fold the waves' sums in wave order; thread 0 stores the workgroup's partials.
template <int NW>
__device__ __forceinline__ void emit_row_sums(const RowSums& s, int lane, int wave,
                                              double* part_loss, double* part_res) {
  __shared__ double lx[NW], rx[NW];
  double wl = s.loss, wr = s.res;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    wl += __shfl_xor(wl, m, 64);
    wr += __shfl_xor(wr, m, 64);
  }
  if (lane == 0) {
    lx[wave] = wl;
    rx[wave] = wr;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double a = 0., b = 0.;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      a += lx[w];
      b += rx[w];
    }
    part_loss[blockIdx.x] = a;
    if (part_res) part_res[blockIdx.x] = b;
  }
}

// What one launch of shard_pass does with a tile.
enum : int {
  kPassFused = 0,  // dot, sigmoid/residual/loss, rank-1 update: X read once
  kPassDot = 1,    // only the partial dot of this column block -> z_buf
  kPassAxpy = 2,   // only the rank-1 update, residual taken from res_in
};

// h, residual's model output and the loss term of one row from z = x.theta
// (reference lr.cpp:69-72 and :325-329; ridge.hpp:105-107 for the identity link)
__device__ __forceinline__ void row_terms(double z, double yv, unsigned loss_mode,
                                          int identity_link, double& h, double& l) {
  if (identity_link) {
    h = z;
  } else {
    const double e = exp(-z);
    h = 1. / (1. + e);
  }
  l = 0.;
  if (loss_mode != kLossNone) {
    if (loss_mode == kLossReference) {
      l = -log((yv == 1.) ? h : 1. - h);
    } else if (loss_mode == kLossSquared) {
      l = (h - yv) * (h - yv);
    } else {
      const double sgn = (yv == 1.) ? -z : z;  // loss = log(1 + exp(sgn))
      l = log1p(exp(-fabs(sgn))) + fmax(sgn, 0.);
    }
  }
}

// Row held by `lane` after the transposing reduction over R rows.
template <int R>
__device__ __forceinline__ int row_of_lane(int lane) {
  int rho = 0;
#pragma unroll
  for (int s = 0; (1 << s) < R; ++s)
    if (lane & (1 << s)) rho += R >> (s + 1);
  return rho;
}

// Lowest lane that holds row r (inverse of row_of_lane on lanes [0, R)).
template <int R>
__host__ __device__ constexpr int lane_of_row(int r) {
  int lane = 0;
  for (int s = 0; (1 << s) < R; ++s)
    if (r & (R >> (s + 1))) lane |= (1 << s);
  return lane;
}

// p[r] = this lane's partial dot of row r.  Returns the full 64-lane sum of
// row row_of_lane<R>(lane); identical bits in every lane holding that row.
constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v >> 1); }

// The partials travel in an ext-vector (pure SSA values): with a plain array
// the compiler folds the lane-dependent selects into dynamically indexed
// loads and parks the array in scratch memory.
template <int R>
struct RowVec {
  typedef double type __attribute__((ext_vector_type(R)));
};
template <>
struct RowVec<1> {
  typedef double type;
};

template <int R>
__device__ __forceinline__ double reduce_rows(typename RowVec<R>::type p, int lane) {
  constexpr int kSteps = ilog2(R);
  double z;
  if constexpr (R == 1) {
    z = p;
  } else {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const int cnt = R >> (s + 1);
      const int m = 1 << s;
      const bool up = (lane & m) != 0;
#pragma unroll
      for (int k = 0; k < cnt; ++k) {
        const double lo = p[k], hi = p[k + cnt];
        const double send = up ? lo : hi;
        const double keep = up ? hi : lo;
        p[k] = keep + __shfl_xor(send, m, kWave);
      }
    }
    z = p[0];
  }
#pragma unroll
  for (int s = kSteps; s < 6; ++s) z += __shfl_xor(z, 1 << s, kWave);
  return z;
}

__device__ __forceinline__ double bcast_lane(double v, int src_lane) {
  // src_lane is a compile-time constant at every call site: two v_readlane.
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __builtin_amdgcn_readlane(lo, src_lane);
  hi = __builtin_amdgcn_readlane(hi, src_lane);
  return __hiloint2double(hi, lo);
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int m = 1; m < kWave; m <<= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

// Per-wave constants of one pass.
struct WaveCtx {
  int lane;
  int wc;             // column slab of this wave within the workgroup
  int my_nch;         // chunks this wave really owns
  int ragged_c;       // its chunk that straddles the row end, or -1
  bool lane_in_ragged;
  int my_row;         // row of the tile whose dot product ends up in this lane
  uint32_t lane_off;  // byte offset of this lane inside a chunk
  // tail stage (TL > 0): this lane's place among the leftover columns
  bool owns_tail;     // this wave handles them (the last one of the workgroup's row)
  bool tail_in;       // ... and the lane's column pair exists
  int tail_row;       // row, within one tail load, that the lane reads
  int tail_slot;      // lane holding the tail dot of row my_row
  uint32_t tail_off;  // byte offset of the lane's pair from the tile base
  int tail_src[4];    // per tail load: lane holding the residual of its row
  double bias;        // theta of the constant first column that is not stored, or 0
};

// Geometry of the tail stage: a tile's R rows are covered by TL loads of
// R/TL rows each, kWave*TL/R adjacent lanes per row.
template <int R, int TL>
struct TailGeo {
  static constexpr int kRowsPerLoad = R / (TL > 0 ? TL : 1);
  static constexpr int kLanesPerRow = kWave / kRowsPerLoad;
};

// Issue every load of one tile of R rows (uniform base + 32-bit lane offset).
// FULL = every row of the tile exists; ALLCH = the wave uses all NCH chunks.
template <int NCH, int R, bool FULL, bool ALLCH, int MODE, int TL>
__device__ __forceinline__ void load_tile(const PassArgs& a, const WaveCtx& w,
                                          const double* tile_base, int64_t row0,
                                          v2d (&x)[R][NCH], v2d (&xt)[TL > 0 ? TL : 1],
                                          double& yv) {
  // The chunk that straddles the row end is loaded whole; compute_tile drops
  // its lanes past the row end.  (Loading it under the lane mask instead, so
  // that those lanes request nothing, was measured on 3 GB shards for every
  // variant: 1-8 % slower from 98 to 3500 columns, whether the masked loads
  // were interleaved with the others of the tile or issued as a group behind
  // them.)
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const char* rowp = reinterpret_cast<const char*>(tile_base + (int64_t)r * a.pitch);
    const bool rv = FULL || (row0 + r) < a.n;  // uniform
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      x[r][c] = v2d{0., 0.};
      if (rv && (ALLCH || c < w.my_nch))  // uniform
        x[r][c] = load_x(reinterpret_cast<const v2d*>(
            rowp + w.lane_off + (uint32_t)(c * kChunkCols * sizeof(double))));
    }
  }
  if constexpr (TL > 0) {
    constexpr int kRpl = TailGeo<R, TL>::kRowsPerLoad;
#pragma unroll
    for (int j = 0; j < TL; ++j) {
      xt[j] = v2d{0., 0.};
      if (w.tail_in && (FULL || row0 + j * kRpl + w.tail_row < a.n))
        xt[j] = load_x(reinterpret_cast<const v2d*>(
            reinterpret_cast<const char*>(tile_base + (int64_t)(j * kRpl) * a.pitch) +
            w.tail_off));
    }
  }
  // the per-row scalar that goes with the tile: the label, or (second sweep
  // of a column-blocked row) the residual
  yv = 0.;
  const double* per_row = (MODE == kPassAxpy) ? a.res_in : a.y;
  if (MODE != kPassDot && (FULL || row0 + w.my_row < a.n) && per_row)
    yv = per_row[row0 + w.my_row];
}

// Everything that happens on a loaded tile: dots, lane reduction,
// sigmoid/residual/loss, rank-1 update of the gradient slab.
// THL: theta is read from the wave's LDS slab (thl) instead of registers.
template <int NCH, int R, int WCOL, bool GRAD, bool FULL, bool THL, int MODE, int TL>
__device__ __forceinline__ void compute_tile(const PassArgs& a, const WaveCtx& w,
                                             int64_t row0, v2d (&x)[R][NCH],
                                             const v2d (&xt)[TL > 0 ? TL : 1], double yv,
                                             const v2d (&th)[NCH], const v2d* thl, v2d tht,
                                             v2d (&acc)[NCH], v2d& acct, RowSums& sums,
                                             double* zbuf, double& h_keep, int64_t& h_row) {
  const int lane = w.lane;
  const int64_t myrow_g = row0 + w.my_row;
  const bool my_valid = FULL || myrow_g < a.n;

  // lanes past the end of the row in the ragged last chunk hold the next
  // row's (or slack) bytes: zero them so they cannot poison the dot product
  if (w.ragged_c >= 0) {
#pragma unroll
    for (int c = 0; c < NCH; ++c)
      if (c == w.ragged_c) {
#pragma unroll
        for (int r = 0; r < R; ++r) x[r][c] = w.lane_in_ragged ? x[r][c] : v2d{0., 0.};
      }
  }

  double res;
  if constexpr (MODE == kPassAxpy) {
    res = my_valid ? yv : 0.;  // yv carries the residual in this sweep
  } else {
    // ---- per-lane partial dots ----
    typename RowVec<R>::type p;
    {
      double s0[R], s1[R];
#pragma unroll
      for (int r = 0; r < R; ++r) s0[r] = s1[r] = 0.;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const v2d t = THL ? thl[c * kWave] : th[c];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          s0[r] = fma(x[r][c].x, t.x, s0[r]);
          s1[r] = fma(x[r][c].y, t.y, s1[r]);
        }
      }
      // one tail load per row (TL == R): all 64 lanes of load r belong to row
      // r, so the leftover columns are simply one more term of the partial
      if constexpr (TL > 0 && TL == R) {
        if (w.owns_tail) {  // uniform
#pragma unroll
          for (int r = 0; r < R; ++r) {
            s0[r] = fma(xt[r].x, tht.x, s0[r]);
            s1[r] = fma(xt[r].y, tht.y, s1[r]);
          }
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if constexpr (R == 1)
          p = s0[r] + s1[r];
        else
          p[r] = s0[r] + s1[r];
      }
    }
    double z = reduce_rows<R>(p, lane);

    if (TL > 0 && TL < R && w.owns_tail) {  // uniform
      // leftover columns: segment sums, then each row's sum to the lane that
      // holds the row
      constexpr int kRpl = TailGeo<R, TL>::kRowsPerLoad;
      constexpr int kLpr = TailGeo<R, TL>::kLanesPerRow;
      double tz = 0.;
#pragma unroll
      for (int j = 0; j < TL; ++j) {
        double t = fma(xt[j].x, tht.x, xt[j].y * tht.y);
#pragma unroll
        for (int m = 1; m < kLpr; m <<= 1) t += __shfl_xor(t, m, kWave);
        const double got = __shfl(t, w.tail_slot, kWave);
        if (TL == 1 || w.my_row / kRpl == j) tz = got;
      }
      z += tz;
    }

    if (WCOL > 1) {
      if (lane < R) zbuf[w.wc * R + w.my_row] = z;
      __syncthreads();
      double s = 0.;
#pragma unroll
      for (int k = 0; k < WCOL; ++k) s += zbuf[k * R + w.my_row];
      z = s;
    }

    if constexpr (MODE == kPassDot) {
      // first sweep of a column-blocked row: only the partial dot leaves
      if (my_valid && lane < R && w.wc == 0)
        a.z_buf[myrow_g] = a.z_accumulate ? a.z_buf[myrow_g] + z : z;
      return;
    }

    // ---- sigmoid, residual, loss for the row this lane holds ----
    double h, l;
    row_terms(z + w.bias, yv, a.loss_mode, a.identity_link, h, l);
    res = my_valid ? (h - yv) : 0.;
    // predictions are not stored here but after the NEXT tile's loads have been
    // issued (see the tile loop): a store in front of them would have to be
    // acknowledged before any of their data counts as returned
    h_keep = h;
    h_row = (my_valid && lane < R && w.wc == 0) ? myrow_g : -1;
    if (my_valid && lane < R && w.wc == 0) {
      sums.loss += l;
      sums.res += res;
    }
  }

  // ---- rank-1 update of the gradient slab from the same registers ----
  if (GRAD) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const double rr = bcast_lane(res, lane_of_row<R>(r));
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        acc[c].x = fma(rr, x[r][c].x, acc[c].x);
        acc[c].y = fma(rr, x[r][c].y, acc[c].y);
      }
      if constexpr (TL > 0 && TL == R) {
        if (w.owns_tail) {  // uniform
          acct.x = fma(rr, xt[r].x, acct.x);
          acct.y = fma(rr, xt[r].y, acct.y);
        }
      }
    }
    if (TL > 0 && TL < R && w.owns_tail) {  // uniform
#pragma unroll
      for (int j = 0; j < TL; ++j) {
        const double rr = __shfl(res, w.tail_src[j], kWave);
        acct.x = fma(rr, xt[j].x, acct.x);
        acct.y = fma(rr, xt[j].y, acct.y);
      }
    }
  }
}

// NCH  : 128-column chunks per wave (compile-time bound; nch_rt used)
// R    : rows per tile (power of two, <= 64)
// WCOL : waves of a workgroup side by side over the columns
// WROW : independent row groups per workgroup (must be 1 when WCOL > 1)
// MINW : waves per SIMD the register allocation must leave room for
// GRAD : accumulate the gradient (false: loss / predict only)
// ALLCH: the row is exactly WCOL*NCH chunks wide (the last one may be ragged),
//        so no wave has an unused chunk slot and no load is predicated
// THL  : theta lives in LDS (one slab per wave) instead of registers -- for
//        wide rows, where theta + accumulators + tile would not fit
// MODE : kPassFused, or one of the two sweeps of a column-blocked row
// TL   : 0, or the number of loads per tile that cover the columns past the
//        WCOL*NCH full chunks (a.tail_cols of them, at most 128*TL/R)
template <int NCH, int R, int WCOL, int WROW, int MINW, bool GRAD, bool ALLCH, bool THL,
          int MODE = kPassFused, int TL = 0>
__global__ __launch_bounds__(kWave* WCOL* WROW, MINW) void shard_pass(PassArgs a) {
  static_assert(WCOL == 1 || WROW == 1, "column-split workgroups own one row group");
  static_assert((R & (R - 1)) == 0 && R <= kWave, "R must be a power of two");
  static_assert(TL == 0 || (ALLCH && MODE == kPassFused && TL <= R && TL <= 4 &&
                            (TL & (TL - 1)) == 0),
                "the tail stage goes with rows of exactly WCOL*NCH full chunks");
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform
  const int wc = (WCOL > 1) ? wave : 0;
  const int wr = (WCOL > 1) ? 0 : wave;

  // with a tail stage the chunks are the WCOL*NCH full ones
  const int64_t chunks = (TL > 0) ? NCH * WCOL : (a.width + kChunkCols - 1) / kChunkCols;
  const int64_t slab_c0 = (int64_t)wc * a.nch_rt;          // first chunk of this wave
  int64_t left = chunks - slab_c0;
  const int my_nch = ALLCH ? NCH : (int)(left < 0 ? 0 : (left > a.nch_rt ? a.nch_rt : left));
  const int64_t slab_col0 = slab_c0 * kChunkCols;
  const int64_t col0 = slab_col0 + 2 * lane;
  // the chunk that straddles the end of the row, if this wave owns it
  const int rag_cols = (TL > 0) ? 0 : (int)(a.width % kChunkCols);
  const int ragged_c = (rag_cols != 0 && slab_c0 + my_nch == chunks && my_nch > 0)
                           ? my_nch - 1 : -1;
  const bool lane_in_ragged = 2 * lane < rag_cols;
  WaveCtx w;
  w.lane = lane;
  w.wc = wc;
  w.my_nch = my_nch;
  w.ragged_c = ragged_c;
  w.lane_in_ragged = lane_in_ragged;
  w.my_row = row_of_lane<R>(lane & (R - 1));
  w.lane_off = (uint32_t)(2 * lane * sizeof(double));
  constexpr int kRpl = TailGeo<R, TL>::kRowsPerLoad;
  constexpr int kLpr = TailGeo<R, TL>::kLanesPerRow;
  constexpr int64_t kBodyCols = (int64_t)NCH * kChunkCols;
  const int tail_pair = lane & (kLpr - 1);
  v2d tht = v2d{0., 0.}, acct = v2d{0., 0.};
  w.owns_tail = TL > 0 && wc == WCOL - 1;  // the wave next to the leftover columns
  if constexpr (TL > 0) {
    w.tail_in = w.owns_tail && 2 * tail_pair < a.tail_cols;
    w.tail_row = lane / kLpr;
    w.tail_slot = (w.my_row % kRpl) * kLpr;
    w.tail_off = (uint32_t)(((int64_t)w.tail_row * a.pitch + kBodyCols + 2 * tail_pair) *
                            sizeof(double));
#pragma unroll
    for (int j = 0; j < TL; ++j) w.tail_src[j] = lane_of_row<R>(j * kRpl + w.tail_row);
    if (w.tail_in)
      tht = *reinterpret_cast<const v2d*>(a.theta + slab_col0 + kBodyCols + 2 * tail_pair);
  }

  // theta slab -> registers, or -> this wave's private LDS slab (theta is
  // zero-padded on the device)
  __shared__ v2d th_lds[THL ? WCOL * WROW * NCH * kWave : 1];
  v2d* thl = th_lds + (THL ? (wave * NCH * kWave + lane) : 0);
  v2d thr[NCH], acc[NCH];  // thr is dead (and eliminated) when THL
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    v2d t = v2d{0., 0.};
    acc[c] = v2d{0., 0.};
    if (ALLCH || c < a.nch_rt)
      t = *reinterpret_cast<const v2d*>(a.theta + col0 + (int64_t)c * kChunkCols);
    if (THL) thl[c * kWave] = t;
    thr[c] = t;
  }
  RowSums sums;
  w.bias = (MODE == kPassFused && a.theta_bias) ? *a.theta_bias : 0.;

  __shared__ double zx[(WCOL > 1) ? 2 * WCOL * R : 1];

  const int64_t group = (int64_t)blockIdx.x * WROW + wr;
  const int64_t ngroups = (int64_t)gridDim.x * WROW;
  const int64_t nfull = a.n / R;  // tiles with all R rows present
  const int64_t tile_stride = (int64_t)R * a.pitch;
  const double* xbase = a.X + slab_col0;
  constexpr int kZ = (WCOL > 1) ? WCOL * R : 0;

  // full tiles, then the one partial tile of the shard (if this row group
  // is the one it falls to)
  int64_t tile = group;
  int par = 0;  // which half of zx the next tile uses (alternates per tile)
  double h_keep = 0.;   // prediction of the previous tile's row in this lane,
  int64_t h_row = -1;   // stored once the current tile's loads are on their way
  auto store_kept = [&]() {
    if (MODE == kPassFused && a.h_out && h_row >= 0) store_h(a.h_out + h_row, h_keep);
  };
#pragma clang loop unroll(disable)
  for (; tile < nfull; tile += ngroups, par ^= 1) {
    v2d x[R][NCH], xt[TL > 0 ? TL : 1];
    double yv;
    load_tile<NCH, R, true, ALLCH, MODE, TL>(a, w, xbase + tile * tile_stride, tile * R, x, xt,
                                             yv);
    store_kept();
    compute_tile<NCH, R, WCOL, GRAD, true, THL, MODE, TL>(a, w, tile * R, x, xt, yv, thr, thl,
                                                          tht, acc, acct, sums,
                                                          zx + par * kZ, h_keep, h_row);
  }
  if (tile < a.ntiles) {
    v2d x[R][NCH], xt[TL > 0 ? TL : 1];
    double yv;
    load_tile<NCH, R, false, ALLCH, MODE, TL>(a, w, xbase + tile * tile_stride, tile * R, x, xt,
                                              yv);
    store_kept();
    compute_tile<NCH, R, WCOL, GRAD, false, THL, MODE, TL>(a, w, tile * R, x, xt, yv, thr, thl,
                                                           tht, acc, acct, sums,
                                                           zx + par * kZ, h_keep, h_row);
  }
  store_kept();

  // ---- combine the workgroup's partials in a fixed order ----
  if (GRAD) {
    double* out = a.part_g + (int64_t)blockIdx.x * a.pitch;
    __shared__ v2d gx[(WROW > 1) ? (WROW - 1) * kWave : 1];
    // one column pair per lane: sum over the workgroup's row groups in wave
    // order (uniform call: every wave of the workgroup passes through)
    auto emit = [&](v2d v, bool mine, double* dst) {
      if (WROW == 1) {
        if (mine) *reinterpret_cast<v2d*>(dst) = v;
      } else {
        if (wr > 0) gx[(wr - 1) * kWave + lane] = v;
        __syncthreads();
        if (wr == 0) {
#pragma unroll
          for (int k = 1; k < WROW; ++k) {
            const v2d o = gx[(k - 1) * kWave + lane];
            v.x += o.x;
            v.y += o.y;
          }
          if (mine) *reinterpret_cast<v2d*>(dst) = v;
        }
        __syncthreads();
      }
    };
#pragma unroll
    for (int c = 0; c < NCH; ++c)
      if (c < my_nch)  // uniform over the workgroup when WROW > 1 (WCOL == 1 there)
        emit(acc[c], c != ragged_c || lane_in_ragged, out + col0 + (int64_t)c * kChunkCols);
    if constexpr (TL > 0) {
      // the leftover columns: fold the row segments of the wave first
#pragma unroll
      for (int m = kLpr; m < kWave; m <<= 1) {
        acct.x += __shfl_xor(acct.x, m, kWave);
        acct.y += __shfl_xor(acct.y, m, kWave);
      }
      emit(acct, lane < kLpr && w.tail_in, out + slab_col0 + kBodyCols + 2 * tail_pair);
    }
  }
  if constexpr (MODE == kPassFused)  // the sweeps of a blocked row carry no loss
    emit_row_sums<WCOL * WROW>(sums, lane, wave, a.part_loss, a.part_res);
}

// ---------------------------------------------------------------------------
// Narrow rows in the row-tiled layout: a lane per row.
//
// The library owns the layout of the shard in HBM, and for rows of at most 64
// columns it stores tiles of 64 rows column pair by column pair:
//   X[((tile * NP + p) * 64 + r) * 2 + {0, 1}] = columns 2p, 2p+1 of row 64*tile + r
// (NP = ceil(d / 2) pairs; an odd d is padded with one zero column, rows are
// padded with zero rows to whole groups of U tiles).  Lane r of a wave then
// owns row r of a tile whatever the width: every load instruction moves a
// dense 1 KiB, the dot product is a chain of FMAs inside the lane in column
// order (the reference's own order, ext_utility.hpp:171-174) with theta
// broadcast from LDS, all 64 lanes evaluate 64 different sigmoid / loss terms,
// labels and predictions are dense 512-byte accesses, and the rank-1 update
// needs no residual exchange.  The per-lane gradient accumulators are summed
// over the lanes once, at the end of the kernel.
//
// Same reference loops as shard_pass (lr.cpp:69-72,132-138,322-330,361-363).
// tile_rows (below) brings uploaded row-major rows into this layout.
template <int NP, int U, int WROW, int MINW, bool GRAD>
__global__ __launch_bounds__(kWave* WROW, MINW) void lane_pass(PassArgs a) {
  static_assert(NP >= 1 && NP <= 32, "lane-per-row tiles hold rows of 2..64 columns");
  const int lane = threadIdx.x & (kWave - 1);
  const int wr = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);

  __shared__ v2d th_lds[NP];
  if (threadIdx.x < NP) th_lds[threadIdx.x] = *reinterpret_cast<const v2d*>(a.theta + 2 * threadIdx.x);
  __syncthreads();
  const double bias = a.theta_bias ? *a.theta_bias : 0.;

  v2d acc[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) acc[p] = v2d{0., 0.};
  RowSums sums;

  constexpr int64_t kGroupRows = (int64_t)kWave * U;
  const int64_t ngroups = (a.n + kGroupRows - 1) / kGroupRows;
  const int64_t stride = (int64_t)gridDim.x * WROW;
  // Software pipeline: the loads of a wave's NEXT group are in flight while it
  // works on this one (two register buffers, the loop unrolled by two).  Every
  // load is unconditional -- past the last group the last group is asked for
  // again and dropped, a row past the end reads the last label -- so the wait
  // for a buffer counts exactly the loads issued after it.  Without labels
  // (predict) the first theta entry stands in for the address.
  const double* ybase = a.y ? a.y : a.theta;
  auto request = [&](int64_t g, v2d (&x)[U][NP], double (&yv)[U]) {
    if (g >= ngroups) g = ngroups - 1;
    const v2d* base = reinterpret_cast<const v2d*>(a.X) + g * (U * NP * kWave) + lane;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int p = 0; p < NP; ++p) x[u][p] = load_x(base + (u * NP + p) * kWave);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int64_t row = g * kGroupRows + lane + u * kWave;
      if (row >= a.n) row = a.n - 1;
      yv[u] = ybase[a.y ? row : 0];
    }
  };
  auto work = [&](int64_t g, v2d (&x)[U][NP], double (&yl)[U]) {
    const int64_t row0 = g * kGroupRows + lane;
    // keeps the theta reads inside the loop: hoisted, they would occupy
    // 4 * NP registers next to x and acc
    asm volatile("" ::: "memory");
#pragma unroll
    for (int u = 0; u < U; ++u) {
      double z = 0.;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const v2d th = th_lds[p];
        z = fma(x[u][p].x, th.x, z);
        z = fma(x[u][p].y, th.y, z);
      }
      const bool valid = row0 + u * kWave < a.n;
      const double yv = a.y ? yl[u] : 0.;
      double h, l;
      row_terms(z + bias, yv, a.loss_mode, a.identity_link, h, l);
      const double res = valid ? (h - yv) : 0.;
      if (valid) {
        sums.loss += l;
        sums.res += res;
      }
      if constexpr (GRAD) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
          acc[p].x = fma(res, x[u][p].x, acc[p].x);
          acc[p].y = fma(res, x[u][p].y, acc[p].y);
        }
      } else {
        // predictions go with the passes that carry no gradient.  A plain store: the
        // destination is device memory here, and letting the L2 write the lines
        // back in its own time is 3.5 % faster than the non-temporal form
        // (30 M x 16: 0.720 against 0.746 ms)
        if (a.h_out && valid) a.h_out[row0 + u * kWave] = h;
      }
    }
  };
  int64_t g = (int64_t)blockIdx.x * WROW + wr;
  if (g < ngroups) {
    v2d xa[U][NP], xb[U][NP];
    double ya[U], yb[U];
    request(g, xa, ya);
#pragma clang loop unroll(disable)
    for (;;) {
      request(g + stride, xb, yb);
      work(g, xa, ya);
      g += stride;
      if (g >= ngroups) break;
      request(g + stride, xa, ya);
      work(g, xb, yb);
      g += stride;
      if (g >= ngroups) break;
    }
  }

  if (GRAD) {
    __shared__ v2d gx[(WROW > 1) ? (WROW - 1) * NP : 1];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      acc[p].x = wave_sum(acc[p].x);
      acc[p].y = wave_sum(acc[p].y);
      if (WROW > 1 && wr > 0 && lane == 0) gx[(wr - 1) * NP + p] = acc[p];
    }
    if (WROW > 1) __syncthreads();
    if (wr == 0 && lane == 0) {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        v2d s = acc[p];
#pragma unroll
        for (int w = 1; w < WROW; ++w) {
          const v2d o = gx[(w - 1) * NP + p];
          s.x += o.x;
          s.y += o.y;
        }
        *reinterpret_cast<v2d*>(a.part_g + (int64_t)blockIdx.x * (2 * NP) + 2 * p) = s;
      }
    }
  }
  emit_row_sums<WROW>(sums, lane, wr, a.part_loss, a.part_res);
}

// Rows row0 .. row0+nrows-1 of the shard as dense row-major rows of d doubles
// (what plr_set_data takes): the inverse of the upload.  np > 0: the shard is
// row-tiled (tile_rows); skip = 1: its constant first column is not stored and
// comes back as 1.0.
__global__ void gather_rows(const double* X, int64_t pitch, int np, int64_t row0, int64_t nrows,
                            int d, int skip, double* dst) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nrows * d) return;
  const int64_t r = i / d;
  const int col = (int)(i % d) - skip;
  const int64_t row = row0 + r;
  double v = 1.;
  if (col >= 0)
    v = np > 0 ? X[((((row / kWave) * np + (col >> 1)) * kWave) + (row % kWave)) * 2 + (col & 1)]
               : X[row * pitch + col];
  dst[i] = v;
}

// Rows row_lo .. row_hi-1 of a row-tiled shard (np column pairs per row) set to
// zero: the rows behind the last one in the last group of tiles, which the
// pass reads and which nobody else has written.
__global__ void zero_tiled_rows(double* X, int np, int64_t row_lo, int64_t row_hi) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = row_lo + i / np;
  const int p = (int)(i % np);
  if (row >= row_hi) return;
  reinterpret_cast<v2d*>(X)[((row / kWave) * np + p) * kWave + (row % kWave)] = v2d{0., 0.};
}

// lane_pass for the wider tiles (34..64 columns), where rows and accumulators
// of a whole tile fill the registers of a wave (one wave per SIMD): a PAIR of
// waves shares every tile, each holding half of the column pairs of the same
// 64 rows, so that twice as many waves fit.  The halves of a row's dot product
// meet in LDS (double-buffered, one barrier per group of tiles; a workgroup is
// one pair, so the barrier couples nobody else) and are added in wave order;
// both waves then evaluate the row terms and update their own columns.
template <int NP, int U, int MINW, bool GRAD>
__global__ __launch_bounds__(2 * kWave, MINW) void lane2_pass(PassArgs a) {
  static_assert(NP >= 2 && NP <= 32, "lane-per-row tiles hold rows of 2..64 columns");
  constexpr int NPW = (NP + 1) / 2;  // column pairs per wave
  const int lane = threadIdx.x & (kWave - 1);
  const int wc = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int p0 = wc * NPW;
  // an odd number of pairs: the second wave's last slot lies past the row
  const bool short_last = (NP & 1) && wc == 1;  // uniform

  __shared__ v2d th_lds[2 * NPW];
  __shared__ double zx[2][2][U][kWave];
  if (threadIdx.x < 2 * NPW)  // theta is zero-padded far beyond the row
    th_lds[threadIdx.x] = *reinterpret_cast<const v2d*>(a.theta + 2 * threadIdx.x);
  __syncthreads();
  const double bias = a.theta_bias ? *a.theta_bias : 0.;

  v2d acc[NPW];
#pragma unroll
  for (int p = 0; p < NPW; ++p) acc[p] = v2d{0., 0.};
  RowSums sums;
  double h_keep[U];
  int64_t h_row0 = -1;
#pragma unroll
  for (int u = 0; u < U; ++u) h_keep[u] = 0.;
  auto store_kept = [&]() {
    if (a.h_out && h_row0 >= 0 && wc == 0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t row = h_row0 + u * kWave;
        if (row < a.n) store_h(a.h_out + row, h_keep[u]);
      }
    }
  };

  constexpr int64_t kGroupRows = (int64_t)kWave * U;
  const int64_t ngroups = (a.n + kGroupRows - 1) / kGroupRows;
  int par = 0;
#pragma clang loop unroll(disable)
  for (int64_t g = blockIdx.x; g < ngroups; g += gridDim.x, par ^= 1) {
    const v2d* base = reinterpret_cast<const v2d*>(a.X) + g * (U * NP * kWave) + p0 * kWave + lane;
    v2d x[U][NPW];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int p = 0; p < NPW; ++p) {
        x[u][p] = v2d{0., 0.};
        if (!(p == NPW - 1 && short_last)) x[u][p] = load_x(base + (u * NP + p) * kWave);
      }
    const int64_t row0 = g * kGroupRows + lane;
    double yv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t row = row0 + u * kWave;
      yv[u] = (a.y && row < a.n) ? a.y[row] : 0.;
    }
    store_kept();
    asm volatile("" ::: "memory");  // keeps the theta reads inside the loop
#pragma unroll
    for (int u = 0; u < U; ++u) {
      double z = 0.;
#pragma unroll
      for (int p = 0; p < NPW; ++p) {
        const v2d th = th_lds[p0 + p];
        z = fma(x[u][p].x, th.x, z);
        z = fma(x[u][p].y, th.y, z);
      }
      zx[par][wc][u][lane] = z;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const double z = zx[par][0][u][lane] + zx[par][1][u][lane];
      const bool valid = row0 + u * kWave < a.n;
      double h, l;
      row_terms(z + bias, yv[u], a.loss_mode, a.identity_link, h, l);
      const double res = valid ? (h - yv[u]) : 0.;
      h_keep[u] = h;
      if (valid && wc == 0) {
        sums.loss += l;
        sums.res += res;
      }
      if (GRAD) {
#pragma unroll
        for (int p = 0; p < NPW; ++p) {
          acc[p].x = fma(res, x[u][p].x, acc[p].x);
          acc[p].y = fma(res, x[u][p].y, acc[p].y);
        }
      }
    }
    h_row0 = row0;
  }
  store_kept();

  if (GRAD) {
#pragma unroll
    for (int p = 0; p < NPW; ++p) {
      acc[p].x = wave_sum(acc[p].x);
      acc[p].y = wave_sum(acc[p].y);
    }
    if (lane == 0) {
#pragma unroll
      for (int p = 0; p < NPW; ++p)
        if (!(p == NPW - 1 && short_last))
          *reinterpret_cast<v2d*>(a.part_g + (int64_t)blockIdx.x * (2 * NP) + 2 * (p0 + p)) = acc[p];
    }
  }
  emit_row_sums<2>(sums, lane, wc, a.part_loss, a.part_res);
}

// Row-major rows (src: nrows x src_pitch doubles, the first `cols` of each
// used) into the row-tiled layout above, as rows row0 .. row0+nrows-1 of the
// shard.  One thread per (row, column pair); columns at or past `cols` are
// written as zeros.  Runs once per uploaded block of rows.
__global__ void tile_rows(const double* src, int64_t src_pitch, int64_t nrows, int cols,
                          double* X, int64_t row0, int np) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  // consecutive threads take consecutive rows of one column pair: the stores
  // of a wave are one dense KiB
  const int64_t blk = i / ((int64_t)kWave * np);       // block of 64 source rows
  const int rem = (int)(i % ((int64_t)kWave * np));
  const int p = rem / kWave, r = rem % kWave;
  const int64_t srow = blk * kWave + r;
  if (srow >= nrows) return;
  const double* sp = src + srow * src_pitch + 2 * p;
  v2d v;
  v.x = (2 * p < cols) ? sp[0] : 0.;
  v.y = (2 * p + 1 < cols) ? sp[1] : 0.;
  const int64_t row = row0 + srow;
  reinterpret_cast<v2d*>(X)[((row / kWave) * np + p) * kWave + (row % kWave)] = v;
}

// ---------------------------------------------------------------------------
// Rows of 65..128 columns, two rows per wave instruction.  With one row per
// load (shard_pass, one chunk) a pass over rows this short is bound by its
// instruction stream, not by HBM: every load, every multiply-add, every lane
// exchange and the whole exp/log sequence are issued per row (or per 16 rows
// with 16 useful lanes) -- about 35 instructions a row, and half of the lanes
// of most of them past the row end.  Here a half-wave owns a row: lane l works
// on row 2g + l/32 of pair g and holds the column pairs (2q, 2q+1) and
// (64+2q, 65+2q), q = l % 32.  A tile is G pairs; the transposing butterfly
// over the 32 lanes of a half leaves every lane with ONE row of the tile (all
// 64 lanes evaluate distinct sigmoid / loss terms when G = 32), the residuals
// travel back inside the half (ds_bpermute) and the rank-1 update runs on the
// loaded registers.  The second load of a pair fetches columns 64.. of both
// rows; its lanes past the row end fetch the next row's first bytes (or the
// slack behind the shard) and take no part in the dot product.
//
// Same reference loops as shard_pass (lr.cpp:69-72,132-138,322-330,361-363).
template <int G, int WROW, int MINW, bool GRAD>
__global__ __launch_bounds__(kWave* WROW, MINW) void pair_pass(PassArgs a) {
  static_assert((G & (G - 1)) == 0 && G >= 2 && G <= 32, "G pairs per tile, a power of two");
  constexpr int kHalf = kWave / 2;
  constexpr int kTileRows = 2 * G;
  const int lane = threadIdx.x & (kWave - 1);
  const int wr = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int half = lane / kHalf;
  const int q = lane & (kHalf - 1);
  const int64_t p = a.pitch;                         // even, 66..128
  const bool hi_in = kWave + 2 * q < p;              // this lane's second column pair exists
  const int my_pair = row_of_lane<G>(q & (G - 1));   // pair whose row ends up in this lane
  const bool owner = q < G;                          // G < 32: lanes q and q + G hold the same row

  const v2d th_lo = *reinterpret_cast<const v2d*>(a.theta + 2 * q);
  const v2d th_hi = *reinterpret_cast<const v2d*>(a.theta + kWave + 2 * q);  // zero past the row
  const double bias = a.theta_bias ? *a.theta_bias : 0.;
  v2d acc_lo = v2d{0., 0.}, acc_hi = v2d{0., 0.};
  RowSums sums;

  const int64_t group = (int64_t)blockIdx.x * WROW + wr;
  const int64_t ngroups = (int64_t)gridDim.x * WROW;
  const int64_t nfull = a.n / kTileRows;
  const int64_t ntiles = (a.n + kTileRows - 1) / kTileRows;
  const uint32_t lane_off = (uint32_t)((half * p + 2 * q) * sizeof(double));
  const uint32_t pair_bytes = (uint32_t)(2 * p * sizeof(double));

  // a tile's predictions are stored after the next tile's loads have been
  // issued: a store in front of them would have to be acknowledged before any
  // of their data counts as returned
  double h_keep = 0.;
  int64_t h_row = -1;
  auto store_kept = [&]() {
    if (a.h_out && h_row >= 0) store_h(a.h_out + h_row, h_keep);
  };

  auto tile_body = [&](int64_t tile, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    const int64_t row0 = tile * kTileRows;
    const char* base = reinterpret_cast<const char*>(a.X + row0 * p) + lane_off;
    v2d xl[G], xh[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      xl[g] = xh[g] = v2d{0., 0.};
      if (FULL || row0 + 2 * g + half < a.n)
        xl[g] = load_x(reinterpret_cast<const v2d*>(base + g * pair_bytes));
    }
    // the second column pair under the lane mask: lanes past the row end
    // request nothing
    if (hi_in) {
#pragma unroll
      for (int g = 0; g < G; ++g)
        if (FULL || row0 + 2 * g + half < a.n)
          xh[g] = load_x(reinterpret_cast<const v2d*>(base + g * pair_bytes + kWave * sizeof(double)));
    }
    store_kept();  // the previous tile's predictions, behind this tile's loads
    const int64_t myrow = row0 + 2 * my_pair + half;
    const bool valid = FULL || myrow < a.n;
    double yv = 0.;
    if (valid && a.y) yv = a.y[myrow];

    typename RowVec<G>::type t;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const double lo = fma(xl[g].x, th_lo.x, xl[g].y * th_lo.y);
      const double hi = fma(xh[g].x, th_hi.x, xh[g].y * th_hi.y);
      t[g] = lo + hi;  // lanes without a second pair hold zeros there
    }
    // transposing butterfly over the 32 lanes of the half
#pragma unroll
    for (int s = 0; s < ilog2(G); ++s) {
      const int cnt = G >> (s + 1);
      const int m = 1 << s;
      const bool up = (lane & m) != 0;
#pragma unroll
      for (int k = 0; k < cnt; ++k) {
        const double lo = t[k], hi = t[k + cnt];
        const double send = up ? lo : hi;
        const double keep = up ? hi : lo;
        t[k] = keep + __shfl_xor(send, m, kWave);
      }
    }
    double z = t[0];
#pragma unroll
    for (int s = ilog2(G); s < 5; ++s) z += __shfl_xor(z, 1 << s, kWave);

    double h, l;
    row_terms(z + bias, yv, a.loss_mode, a.identity_link, h, l);
    const double res = valid ? (h - yv) : 0.;
    h_keep = h;
    h_row = (valid && owner) ? myrow : -1;
    if (valid && owner) {
      sums.loss += l;
      sums.res += res;
    }
    if (GRAD) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        // the residual of row 2g + half sits in the lane of this half that kept pair g
        const double rr = __shfl(res, (lane & kHalf) | lane_of_row<G>(g), kWave);
        acc_lo.x = fma(rr, xl[g].x, acc_lo.x);
        acc_lo.y = fma(rr, xl[g].y, acc_lo.y);
        acc_hi.x = fma(rr, xh[g].x, acc_hi.x);
        acc_hi.y = fma(rr, xh[g].y, acc_hi.y);
      }
    }
  };

  int64_t tile = group;
#pragma clang loop unroll(disable)
  for (; tile < nfull; tile += ngroups) tile_body(tile, std::true_type{});
  if (tile < ntiles) tile_body(tile, std::false_type{});
  store_kept();

  if (GRAD) {
    // the two halves worked on different rows of the same columns
    acc_lo.x += __shfl_xor(acc_lo.x, kHalf, kWave);
    acc_lo.y += __shfl_xor(acc_lo.y, kHalf, kWave);
    acc_hi.x += __shfl_xor(acc_hi.x, kHalf, kWave);
    acc_hi.y += __shfl_xor(acc_hi.y, kHalf, kWave);
    __shared__ v2d gx[(WROW > 1) ? (WROW - 1) * kWave : 1];
    if (WROW > 1) {
      if (wr > 0 && half == 0) {
        gx[(wr - 1) * kWave + q] = acc_lo;
        gx[(wr - 1) * kWave + kHalf + q] = acc_hi;
      }
      __syncthreads();
    }
    if (wr == 0 && half == 0) {
      v2d lo = acc_lo, hi = acc_hi;
#pragma unroll
      for (int k = 1; k < WROW; ++k) {
        const v2d ol = gx[(k - 1) * kWave + q], oh = gx[(k - 1) * kWave + kHalf + q];
        lo.x += ol.x;
        lo.y += ol.y;
        hi.x += oh.x;
        hi.y += oh.y;
      }
      double* out = a.part_g + (int64_t)blockIdx.x * p;
      *reinterpret_cast<v2d*>(out + 2 * q) = lo;
      if (hi_in) *reinterpret_cast<v2d*>(out + kWave + 2 * q) = hi;
    }
  }
  emit_row_sums<WROW>(sums, lane, wr, a.part_loss, a.part_res);
}

// ---------------------------------------------------------------------------
// Rows wider than the fused variants hold (19456 columns), read ONCE.  A team
// of B workgroups shares every row it processes: workgroup b of the team owns
// column block b -- 8 waves side by side, theta of the block in LDS, the
// block's gradient accumulators in registers, one row per step.  What a row
// needs from the other blocks is one number, its partial dot product.  Each
// workgroup publishes its partial in global memory and picks up the others';
// all B workgroups add the B partials in block order, so they arrive at the
// same bits and the team behaves like one very wide workgroup.
//
// Software pipeline, per workgroup, at step t (LAG = 1 or 2 steps between a
// row's dot product and its update):
//     look for the partners' partials of row t - LAG (published LAG steps ago)
//     request row t + 1 into the buffer row t - LAG - 1 has left
//     dot product of row t (requested a whole step ago), wave by wave
//     wave 0 waits until the partners' partials of row t - LAG are all there
//     -- the step's one barrier --
//     publish the partial of row t
//     residual of row t - LAG, rank-1 update from the registers that still hold it
// (One barrier serves both hand-overs inside the workgroup, the waves' partial
// dots to the publishing thread and the partners' partials to everybody: what
// wave 0 waits for in front of it was published LAG steps ago and does not
// depend on this step's partial.  With a barrier for each, 50000 columns ran
// at 0.83 of peak instead of 0.86 and 524288 at 0.77 instead of 0.81.)
// so neither the exchange nor HBM latency stalls the stream: LAG + 2 row
// buffers of NCH chunks per wave rotate.
//
// The exchange needs no fence: a partial travels as two 64-bit words, each
// carrying 32 bits of the double and the 32-bit sequence number of its row
// (never 0; the slots are zeroed before every launch), written and read with
// relaxed device-scope atomics -- a word is valid exactly when its sequence
// number is the expected one.  The slots of a team rotate, and 2 * LAG + 2 of
// them are enough: a workgroup publishes row t only after it has seen every
// partner's partial of row t - LAG - 1, and a partner that has published that
// one still has to read the rows from t - 2 * LAG - 1 on -- so row t may
// overwrite row t - 2 * LAG - 2 and nothing younger.  All workgroups
// of the grid must be resident at once (the host sizes the grid to the
// device); should a partner never show up, the wait gives up after spin_limit
// polls, raises status[0], and every workgroup then runs to its end without
// waiting -- the host reports the pass as failed.
//
// What leaves the kernel besides the gradient partials is z = x.theta of every
// row (z_out): the loss terms, the predictions and the sum of the residuals are
// produced from z by residual_pass, which costs 16 bytes per row against the
// row's 8 * d -- so the kernel carries no log, no loss formula and no
// prediction store, only the link (the sigmoid's exp and division, or
// nothing).  The passes without a gradient need no exchange at all: team_dot
// below.
//
// Same reference loops as shard_pass (lr.cpp:69-72,132-138,322-330,361-363).
constexpr int kTeamWaves = 8;
constexpr int kTeamSlots = 8;  // >= 2 * LAG + 2 for LAG <= 2, a power of two
constexpr int kTeamMaxBlocks = 64;

struct TeamArgs {
  const double* X;
  const double* y;
  const double* theta;       // zero-padded to nblk * blk_chunks * 128 entries
  const double* zeros;       // 128 doubles of zeros (what an unowned chunk slot reads)
  double* part_g;            // [nteams][pitch]
  double* z_out;             // team_pass: n, x.theta per row (without theta_bias);
                             // team_dot: [nblk * 8][nteams][zstride], every wave's
                             // partial of it, a team's rows side by side
  int64_t zstride;           // team_dot: entries per (wave, team), a multiple of 64
  int64_t n, pitch;
  int nblk;                  // B: column blocks = workgroups per team (<= kTeamMaxBlocks)
  int nteams;                // grid = nteams * nblk
  // The row's chunks are dealt evenly: the first blk_extra blocks own
  // blk_chunks + 1 of them, the others blk_chunks; inside a block of m chunks
  // the first m % 8 waves own m / 8 + 1, the others m / 8 -- so no two waves of
  // a team differ by more than two chunks, and none owns more than NCH.
  int blk_chunks;
  int blk_extra;
  const double* theta_bias;  // as in PassArgs
  unsigned long long* zx;    // [nteams][kTeamSlots][nblk][2] exchange slots
  unsigned* status;          // [0]: set when a wait gave up
  unsigned spin_limit;
};

template <int NCH, bool IDENT, int LAG>
__global__ __launch_bounds__(kWave* kTeamWaves, 2) void team_pass(TeamArgs a) {
  static_assert(LAG == 1 || LAG == 2, "a row's update follows its dot product by 1 or 2 steps");
  static_assert(kTeamSlots >= 2 * LAG + 2 && (kTeamSlots & (kTeamSlots - 1)) == 0, "slot ring");
  // Row buffers: rows t - LAG .. t + 1.  (With LAG = 1 a fourth buffer -- row
  // t + 2 in flight as well -- was measured and is 0.5-1 % slower at every
  // width: the step does not wait for data once the waits below are right.)
  constexpr int D = LAG + 2;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  // A team is nblk consecutive workgroups.  Consecutive workgroup ids go to
  // consecutive XCDs, so its members sit on different XCDs and meet in memory,
  // not in an L2 -- the exchange has a whole step to complete, and measured
  // against teams kept inside one XCD this is faster at every width (+1 % at
  // 32768 columns, +9 % at 65536 with the same number of teams), besides
  // leaving no compute unit idle where nblk does not divide an XCD's 32.
  const int blk = (int)(blockIdx.x % a.nblk);
  const int team = (int)(blockIdx.x / a.nblk);

  // my block's chunks, then my wave's share of them
  const int64_t total_chunks = (a.pitch + kChunkCols - 1) / kChunkCols;
  const int blk_m = a.blk_chunks + (blk < a.blk_extra ? 1 : 0);
  const int64_t blk_c0 = (int64_t)blk * a.blk_chunks + (blk < a.blk_extra ? blk : a.blk_extra);
  const int wq = blk_m / kTeamWaves, wrem = blk_m % kTeamWaves;
  const int my_nch = wq + (wave < wrem ? 1 : 0);                       // <= NCH (host-checked)
  const int64_t c0 = blk_c0 + (int64_t)wave * wq + (wave < wrem ? wave : wrem);  // my first chunk
  // the row's last chunk may be ragged (the pitch is a multiple of 16, not of 128)
  const int rag_cols = (int)(a.pitch % kChunkCols);
  const int ragged_c =
      (rag_cols != 0 && my_nch > 0 && c0 + my_nch == total_chunks) ? my_nch - 1 : -1;
  const bool lane_in_ragged = 2 * lane < rag_cols;

  __shared__ v2d th_lds[kTeamWaves * NCH * kWave];
  __shared__ double zw[2][kTeamWaves];        // per-wave partial dots, double-buffered
  __shared__ double zp[2][kTeamMaxBlocks];    // the team's partials of a row, double-buffered
  v2d* thl = th_lds + wave * NCH * kWave + lane;
  v2d acc[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    acc[c] = v2d{0., 0.};
    // (a slot this wave does not own reads the page of zeros: a scalar select, no branch)
    const double* tp = (c < my_nch) ? a.theta + (c0 + c) * kChunkCols : a.zeros;
    thl[c * kWave] = *reinterpret_cast<const v2d*>(tp + 2 * lane);
  }
  const double bias = a.theta_bias ? *a.theta_bias : 0.;
  bool gave_up = false;

  // Uniform base + 32-bit lane offset: no address registers per chunk.  A chunk
  // slot this wave does not own (c >= my_nch) reads a page of zeros instead --
  // a scalar select of the base, so the loop body has no branch per chunk.  The
  // ragged chunk is loaded whole; its lanes past the row end (the next row's
  // bytes) are dropped in the dot product and never stored.
  const char* xwave = reinterpret_cast<const char*>(a.X + c0 * kChunkCols);
  const char* zeros = reinterpret_cast<const char*>(a.zeros);
  const uint32_t lane_off = (uint32_t)(lane * sizeof(v2d));
  const int64_t row_bytes = a.pitch * (int64_t)sizeof(double);
  const int64_t myrows = a.n > team ? (a.n - team + a.nteams - 1) / a.nteams : 0;

  v2d X[D][NCH];
  // Row i of this team -> buf.  Past the team's last row the last row is asked
  // for again (and never used): every step then issues the same loads, with no
  // branch around them, so the wait for row t counts exactly the loads issued
  // after it -- behind a conditional request the compiler has to wait for
  // everything outstanding, the row just requested included.
  auto request = [&](int64_t i, v2d (&buf)[NCH]) {
    if (i >= myrows) i = myrows - 1;
    const char* rp = xwave + (team + i * a.nteams) * row_bytes;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const char* base = (c < my_nch) ? rp + c * (int)(kChunkCols * sizeof(double)) : zeros;
      buf[c] = load_x(reinterpret_cast<const v2d*>(base + lane_off));
    }
  };

  auto step = [&](int64_t t, auto phase_tag) {
    constexpr int PH = decltype(phase_tag)::value;      // t mod D
    constexpr int PREV = (PH + 2) % D;                  // buffer of row t - LAG
    constexpr int NEXT = (PH + 1) % D;                  // buffer of row t - LAG - 1: refilled with t + 1
    const int par = (int)(t & 1);
    const bool have_row = t < myrows;                   // uniform
    const bool have_prev = t >= LAG;                    // uniform

    // Wave 0 collects the partials of row t - LAG (its own included: one code
    // path) with vector loads, and vector loads return in issue order: the
    // first look is requested BEFORE the next row, so it is not queued behind
    // X; any further look comes after it, at the pace rows arrive.
    const bool poller = have_prev && wave == 0 && lane < a.nblk;
    const unsigned seq = (unsigned)(t - LAG + 1);  // sequence number of row t - LAG
    const unsigned long long* pslot =
        a.zx + ((int64_t)(team * kTeamSlots + (int)((t + kTeamSlots - LAG) % kTeamSlots)) * a.nblk +
                (poller ? lane : 0)) * 2;
    unsigned long long w0 = 0, w1 = 0;
    if (poller) {
      w0 = __hip_atomic_load(pslot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      w1 = __hip_atomic_load(pslot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // the label of row t - LAG, for the same reason ahead of the row request:
    // asked for where it is used, it would come back behind row t + 1 and the
    // update would wait for that whole row
    const int64_t prev_row = team + (have_prev ? t - LAG : 0) * a.nteams;
    const double yv = *(a.y ? a.y + prev_row : a.zeros);
    asm volatile("" ::: "memory");
    request(t + 1, X[NEXT]);
    asm volatile("" ::: "memory");

    if (have_row) {
      double s0 = 0., s1 = 0.;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const v2d th = thl[c * kWave];
        const bool drop = (c == ragged_c) && !lane_in_ragged;
        s0 = fma(drop ? 0. : X[PH][c].x, th.x, s0);
        s1 = fma(drop ? 0. : X[PH][c].y, th.y, s1);
      }
      const double wsum = wave_sum(s0 + s1);
      if (lane == 0) zw[par][wave] = wsum;
    }
    // Wave 0 waits for the partners' partials of row t - LAG before the step's
    // one barrier: they were published LAG steps ago and do not depend on this
    // workgroup's partial of row t, which goes out right behind the barrier.
    if (poller) {
      unsigned spins = 0;
      while ((unsigned)(w0 >> 32) != seq || (unsigned)(w1 >> 32) != seq) {
        if (gave_up || spins >= a.spin_limit ||
            ((spins & 63u) == 63u &&
             __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
          gave_up = true;
          __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        ++spins;
        __builtin_amdgcn_s_sleep(2);
        w0 = __hip_atomic_load(pslot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w1 = __hip_atomic_load(pslot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      zp[par][lane] = __longlong_as_double((long long)((w0 & 0xffffffffull) | (w1 << 32)));
    }
    __syncthreads();
    if (have_row && threadIdx.x == 0) {
      double zb = 0.;
#pragma unroll
      for (int w = 0; w < kTeamWaves; ++w) zb += zw[par][w];
      unsigned long long* slot =
          a.zx + ((int64_t)(team * kTeamSlots + (int)(t % kTeamSlots)) * a.nblk + blk) * 2;
      const unsigned long long bits = (unsigned long long)__double_as_longlong(zb);
      const unsigned long long tag = (unsigned long long)(unsigned)(t + 1) << 32;
      __hip_atomic_store(slot, tag | (bits & 0xffffffffull), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slot + 1, tag | (bits >> 32), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    if (have_prev) {
      double z = 0.;
      for (int b = 0; b < a.nblk; ++b) z += zp[par][b];
      if (blk == 0 && threadIdx.x == 0) a.z_out[prev_row] = z;
      // lr.cpp:69-72 / ridge.hpp:79: the model's output, then the residual
      double h = z + bias;
      if (!IDENT) h = 1. / (1. + exp(-h));
      const double res = h - yv;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        acc[c].x = fma(res, X[PREV][c].x, acc[c].x);
        acc[c].y = fma(res, X[PREV][c].y, acc[c].y);
      }
    }
  };

  // Row 0 is requested up front; step t requests row t + 1 first thing.
  // Steps 0 .. myrows + LAG - 1: the last LAG only finish rows.
  if (myrows > 0) {
    request(0, X[0]);
    const int64_t nsteps = myrows + LAG;
    int64_t t = 0;
    if constexpr (D == 3) {
#pragma clang loop unroll(disable)
      for (; t + 3 <= nsteps; t += 3) {
        step(t, std::integral_constant<int, 0>{});
        step(t + 1, std::integral_constant<int, 1>{});
        step(t + 2, std::integral_constant<int, 2>{});
      }
      if (t < nsteps) step(t++, std::integral_constant<int, 0>{});
      if (t < nsteps) step(t++, std::integral_constant<int, 1>{});
    } else {
#pragma clang loop unroll(disable)
      for (; t + 4 <= nsteps; t += 4) {
        step(t, std::integral_constant<int, 0>{});
        step(t + 1, std::integral_constant<int, 1>{});
        step(t + 2, std::integral_constant<int, 2>{});
        step(t + 3, std::integral_constant<int, 3>{});
      }
      if (t < nsteps) step(t++, std::integral_constant<int, 0>{});
      if (t < nsteps) step(t++, std::integral_constant<int, 1>{});
      if (t < nsteps) step(t++, std::integral_constant<int, 2>{});
    }
  }

  double* out = a.part_g + (int64_t)team * a.pitch + c0 * kChunkCols + 2 * lane;
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (c < my_nch && (c != ragged_c || lane_in_ragged))
      *reinterpret_cast<v2d*>(out + (int64_t)c * kChunkCols) = acc[c];
}

// The passes over such rows that carry no gradient (loss only, predictions)
// need nothing from a row but z = x.theta, and no workgroup needs another
// one's share of it: same split of the row over teams of workgroups and their
// waves, but every wave just streams its chunks of its team's rows and stores
// its partial dot products -- kept in the lanes for 64 rows, then written as one
// dense 512-byte store to z_out[((blk * 8 + wave) * nteams + team) * zstride + i],
// i counting the team's rows.  No exchange and no residency requirement.  residual_pass adds a row's partials --
// first over the waves of a block, then over the blocks, the order team_pass
// adds them in, so both give the same bits -- and turns z into loss terms and
// predictions.  Three row buffers rotate: rows t + 1 and t + 2 are in flight
// while row t is summed.
template <int NCH>
__global__ __launch_bounds__(kWave* kTeamWaves, 2) void team_dot(TeamArgs a) {
  constexpr int D = 3;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int blk = (int)(blockIdx.x % a.nblk);
  const int team = (int)(blockIdx.x / a.nblk);
  const int64_t total_chunks = (a.pitch + kChunkCols - 1) / kChunkCols;
  const int blk_m = a.blk_chunks + (blk < a.blk_extra ? 1 : 0);
  const int64_t blk_c0 = (int64_t)blk * a.blk_chunks + (blk < a.blk_extra ? blk : a.blk_extra);
  const int wq = blk_m / kTeamWaves, wrem = blk_m % kTeamWaves;
  const int my_nch = wq + (wave < wrem ? 1 : 0);
  const int64_t c0 = blk_c0 + (int64_t)wave * wq + (wave < wrem ? wave : wrem);
  const int rag_cols = (int)(a.pitch % kChunkCols);
  const int ragged_c =
      (rag_cols != 0 && my_nch > 0 && c0 + my_nch == total_chunks) ? my_nch - 1 : -1;
  const bool lane_in_ragged = 2 * lane < rag_cols;

  v2d th[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const double* tp = (c < my_nch) ? a.theta + (c0 + c) * kChunkCols : a.zeros;
    th[c] = *reinterpret_cast<const v2d*>(tp + 2 * lane);
    if (c == ragged_c && !lane_in_ragged) th[c] = v2d{0., 0.};
  }
  const char* xwave = reinterpret_cast<const char*>(a.X + c0 * kChunkCols);
  const char* zeros = reinterpret_cast<const char*>(a.zeros);
  const uint32_t lane_off = (uint32_t)(lane * sizeof(v2d));
  const int64_t row_bytes = a.pitch * (int64_t)sizeof(double);
  const int64_t myrows = a.n > team ? (a.n - team + a.nteams - 1) / a.nteams : 0;
  double* zmine = a.z_out + ((int64_t)(blk * kTeamWaves + wave) * a.nteams + team) * a.zstride;
  double keep = 0.;  // lane j: this wave's partial of the team's row 64 * (t / 64) + j

  v2d X[D][NCH];
  // unconditional loads, as in team_pass: past the last row the last row again
  auto request = [&](int64_t i, v2d (&buf)[NCH]) {
    if (i >= myrows) i = myrows - 1;
    const char* rp = xwave + (team + i * a.nteams) * row_bytes;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const char* base = (c < my_nch) ? rp + c * (int)(kChunkCols * sizeof(double)) : zeros;
      buf[c] = load_x(reinterpret_cast<const v2d*>(base + lane_off));
    }
  };
  auto step = [&](int64_t t, auto phase_tag) {
    constexpr int PH = decltype(phase_tag)::value;  // t mod 3
    // Nothing is exchanged here: the barrier only keeps the block's eight waves
    // at the same row, so that together they ask for one contiguous piece of it
    // (measured: 6.64 -> 6.73 TB/s at 20000 to 131072 columns).  Every wave of
    // the block takes the same number of steps.
    __builtin_amdgcn_s_barrier();
    request(t + 2, X[(PH + 2) % D]);
    asm volatile("" ::: "memory");
    // the ragged chunk's lanes past the row end hold the next row's bytes: their
    // theta is zero, but a non-finite neighbour must not turn 0 * x into NaN
    double s0 = 0., s1 = 0.;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const bool drop = (c == ragged_c) && !lane_in_ragged;
      s0 = fma(drop ? 0. : X[PH][c].x, th[c].x, s0);
      s1 = fma(drop ? 0. : X[PH][c].y, th[c].y, s1);
    }
    const double wsum = wave_sum(s0 + s1);
    if (lane == (int)(t & (kWave - 1))) keep = wsum;
    if ((t & (kWave - 1)) == kWave - 1 || t == myrows - 1)  // uniform; zstride covers whole groups
      zmine[(t & ~(int64_t)(kWave - 1)) + lane] = keep;
  };
  if (myrows > 0) {
    request(0, X[0]);
    request(1, X[1]);
    int64_t t = 0;
#pragma clang loop unroll(disable)
    for (; t + 3 <= myrows; t += 3) {
      step(t, std::integral_constant<int, 0>{});
      step(t + 1, std::integral_constant<int, 1>{});
      step(t + 2, std::integral_constant<int, 2>{});
    }
    if (t < myrows) step(t++, std::integral_constant<int, 0>{});
    if (t < myrows) step(t++, std::integral_constant<int, 1>{});
  }
}

// Pure streaming read of a buffer with shard_pass's access pattern (a wave
// takes contiguous 8 KiB tiles, interleaved over the grid) and next to no
// arithmetic: what it sustains is the read ceiling the fused pass is up
// against on this device.
__global__ __launch_bounds__(256) void read_probe(const v2d* base, int64_t ntiles, double* sink) {
  constexpr int kLoads = 8;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t group = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t ngroups = (int64_t)gridDim.x * 4;
  v2d acc = v2d{0., 0.};
  for (int64_t t = group; t < ntiles; t += ngroups) {
    const v2d* p = base + t * (kLoads * kWave) + lane;
    v2d x[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) x[i] = load_x(p + i * kWave);
#pragma unroll
    for (int i = 0; i < kLoads; ++i) acc += x[i];
  }
  if (acc.x + acc.y == 1.2345e300) sink[0] = acc.x;  // keeps the loads alive
}

// z = x.theta of every row -> h, residual, loss term, prediction.  Runs between
// the two sweeps of a column-blocked row and behind a team pass.  One thread
// per row, grid-stride; each thread adds its rows' loss terms in the order it
// meets them, the workgroup folds them in a fixed order into part_loss[block]
// (and the residuals into part_res[block]: the gradient of a constant first
// column that is not stored).
// zparts > 0: z[] holds team_dot's partial dot products, [zparts * 8][nteams]
// [zstride], entry i of team m belonging to row m + i * nteams; the threads then
// walk (team, i) so that their reads of z are dense, and a row's z is the sum
// over the zparts groups of the sums over each group's 8 waves, in that order.
__global__ __launch_bounds__(256) void residual_pass(const double* __restrict__ z,
                                                     const double* __restrict__ y,
                                                     double* __restrict__ res,
                                                     double* __restrict__ h_out,
                                                     double* __restrict__ part_loss, int64_t n,
                                                     unsigned loss_mode, int identity_link,
                                                     const double* __restrict__ theta_bias,
                                                     double* __restrict__ part_res, int zparts,
                                                     int nteams, int64_t zstride) {
  const double bias = theta_bias ? *theta_bias : 0.;
  RowSums sums;
  const int64_t count = zparts > 0 ? (int64_t)nteams * zstride : n;
  for (int64_t q = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; q < count;
       q += (int64_t)gridDim.x * blockDim.x) {
    int64_t i = q;
    double zi;
    if (zparts > 0) {
      i = q / zstride + (q % zstride) * nteams;
      if (i >= n) continue;
      zi = 0.;
      for (int b = 0; b < zparts; ++b) {
        const double* zp = z + (int64_t)b * kTeamWaves * count + q;
        double zb = 0.;
#pragma unroll
        for (int w = 0; w < kTeamWaves; ++w) zb += zp[(int64_t)w * count];
        zi += zb;
      }
    } else {
      zi = z[i];
    }
    const double yv = y ? y[i] : 0.;
    double h, l;
    row_terms(zi + bias, yv, loss_mode, identity_link, h, l);
    if (res) res[i] = h - yv;
    if (h_out) store_h(h_out + i, h);
    sums.loss += l;
    sums.res += h - yv;
  }
  emit_row_sums<4>(sums, threadIdx.x & (kWave - 1), threadIdx.x / kWave, part_loss, part_res);
}

// theta arrives in pinned, device-mapped host memory; this one-workgroup
// kernel moves it into the zero-padded device copy the pass reads.  A kernel
// on the pass's own stream instead of a copy command: no hand-over between
// the copy engine and the compute queue in front of every step.
// skip = 1: host_theta[0] belongs to the constant first column, which the
// shard does not store; it goes to dev_theta[bias_slot] and the rest moves up.
__global__ __launch_bounds__(256) void stage_theta(const double* __restrict__ host_theta,
                                                   double* __restrict__ dev_theta, int64_t d,
                                                   int skip, int64_t bias_slot) {
  for (int64_t i = threadIdx.x + (int64_t)blockIdx.x * blockDim.x; i < d - skip;
       i += (int64_t)gridDim.x * blockDim.x)
    dev_theta[i] = host_theta[i + skip];
  if (skip && blockIdx.x == 0 && threadIdx.x == 0) dev_theta[bias_slot] = host_theta[0];
}

// theta already on the device -> the zero-padded copy the pass reads: entries
// [d, len) are written as zeros every time, so a buffer that is shared between
// calls of different widths never leaks an old theta into the pad columns.
__global__ __launch_bounds__(256) void stage_theta_padded(const double* __restrict__ src,
                                                          double* __restrict__ dst, int64_t d,
                                                          int64_t len) {
  for (int64_t i = threadIdx.x + (int64_t)blockIdx.x * blockDim.x; i < len;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = i < d ? src[i] : 0.;
}

// Plain fill with zeros (a kernel, not a memset command: safe inside a
// captured graph).
__global__ __launch_bounds__(256) void fill_zero(double* __restrict__ dst, int64_t count) {
  for (int64_t i = threadIdx.x + (int64_t)blockIdx.x * blockDim.x; i < count;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = 0.;
}

struct FinishArgs {
  const double* part_g;   // [nparts][pitch]
  const double* part_loss;  // [nparts]
  const double* theta;
  double* out;            // the gradient (or delta) of every column, then the loss sum
  int64_t pitch;
  int64_t d;              // stored columns: part_g[.][0 .. d)
  int64_t n;
  // a constant first column that is not stored (PassArgs::theta_bias): its
  // gradient is the sum of the residuals (part_res), its theta sits in
  // *theta_bias; the stored columns then land at out[1 ..], the loss at out[d + 1]
  const double* part_res;  // [nparts_loss], or nullptr
  double* theta_bias;
  int nparts;             // rows of part_g
  int nparts_loss;        // entries of part_loss
  int delta_mode;         // 0: out = gsum; 1: out = -alpha*gsum - coff2*n*theta;
                          // 2: as 1, and theta_rw += delta (the server-side add,
                          //    done in place on the device copy of theta)
  int have_grad;
  double* theta_rw;       // delta_mode 2 only: the device theta to update
  double* loss_slot;      // nullable: also store the loss sum here
  double alpha;
  double coff2;
  // nullable, host memory the device can write: block b stores `seq` to done[b]
  // when everything it writes to `out` has been written (a host thread that
  // polls these words has the results without waiting for the stream to drain)
  unsigned long long* done;
  unsigned long long seq;
  // nullable: a team pass's give-up word (device memory) and where to leave a
  // copy of it for the host (host memory the device can write), so that the
  // host need not fetch it with a copy of its own after every pass
  const unsigned* status_in;
  unsigned long long* status_out;
};

constexpr int kFinCols = 16;
constexpr int kFinSlices = 64;

// Sums the per-workgroup partials: thread (col, slice) adds parts slice,
// slice+64, ... in order (a short chain: the kernel is bound by load latency,
// not bandwidth); the 64 slice sums meet in LDS and are added in slice order.
// Block 0 also folds the loss partials the same way.
__global__ __launch_bounds__(kFinCols* kFinSlices) void finish_pass(FinishArgs a) {
  __shared__ double sm[kFinSlices][kFinCols];
  const int cx = threadIdx.x % kFinCols;
  const int sl = threadIdx.x / kFinCols;
  const int64_t col = (int64_t)blockIdx.x * kFinCols + cx;
  if (a.have_grad) {
    double s = 0.;
    if (col < a.d) {
#pragma unroll 4
      for (int p = sl; p < a.nparts; p += kFinSlices)
        s += a.part_g[(int64_t)p * a.pitch + col];
    }
    sm[sl][cx] = s;
    __syncthreads();
    if (sl == 0 && col < a.d) {
      double g = sm[0][cx];
#pragma unroll
      for (int k = 1; k < kFinSlices; ++k) g += sm[k][cx];
      if (a.delta_mode) {
        const double th = a.theta[col];
        g = -a.alpha * g - (a.coff2 * (double)a.n) * th;
        if (a.delta_mode == 2) a.theta_rw[col] = th + g;  // this thread owns column col
      }
      a.out[col + (a.part_res ? 1 : 0)] = g;
    }
    __syncthreads();
  }
  if (blockIdx.x == 0) {
    double s = 0.;
    for (int p = threadIdx.x; p < a.nparts_loss; p += kFinCols * kFinSlices)
      s += a.part_loss[p];
    sm[sl][cx] = s;
    __syncthreads();
    if (threadIdx.x < kWave) {  // the whole first wave: wave_sum needs all 64 lanes
      const double* flat = &sm[0][0];
      double t = flat[threadIdx.x];
#pragma unroll
      for (int k = 1; k < kFinCols * kFinSlices / kWave; ++k) t += flat[threadIdx.x + k * kWave];
      t = wave_sum(t);
      if (threadIdx.x == 0) {
        a.out[a.d + (a.part_res ? 1 : 0)] = t;
        if (a.loss_slot) *a.loss_slot = t;
      }
    }
    if (a.part_res && a.have_grad) {  // the unstored constant column: same fold over its partials
      __syncthreads();
      double r = 0.;
      for (int p = threadIdx.x; p < a.nparts_loss; p += kFinCols * kFinSlices) r += a.part_res[p];
      sm[sl][cx] = r;
      __syncthreads();
      if (threadIdx.x < kWave) {
        const double* flat = &sm[0][0];
        double t = flat[threadIdx.x];
#pragma unroll
        for (int k = 1; k < kFinCols * kFinSlices / kWave; ++k) t += flat[threadIdx.x + k * kWave];
        t = wave_sum(t);
        if (threadIdx.x == 0) {
          double g = t;
          if (a.delta_mode) {
            const double th = *a.theta_bias;
            g = -a.alpha * g - (a.coff2 * (double)a.n) * th;
            if (a.delta_mode == 2) *a.theta_bias = th + g;
          }
          a.out[0] = g;
        }
      }
    }
  }
  if (a.status_in && blockIdx.x == 0 && threadIdx.x == 0) *a.status_out = *a.status_in;
  if (a.done) {
    __syncthreads();  // every store of this block to `out` has been issued ...
    if (threadIdx.x == 0)  // ... and is visible to the host before the word is
      __hip_atomic_store(a.done + blockIdx.x, a.seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

}  // namespace plr

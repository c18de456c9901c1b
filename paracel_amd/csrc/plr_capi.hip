// C ABI (include/plr.h) over the gfx950 shard kernels: context, resident
// shard, variant selection, launches.  Host C++ only sees plain pointers and
// sizes; nothing here falls back to a CPU path -- if HIP fails, the call
// fails.
#include "../../include/plr.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <functional>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "plr_csv.hpp"
#include "plr_kernels.hpp"
#include "plr_plan.hpp"

struct plr_ctx;
struct CopyPiece {  // bytes of pageable host memory and where on the device they go
  void* dev;
  const void* src;
  size_t bytes;
};
// Host memory moves to and from the device through kCopyLanes lanes of pinned
// staging blocks (see lanes_in / copy_rows_out below).
constexpr int kCopyLanes = 8;
constexpr size_t kCopyBlock = 4u << 20;
struct InJob {  // one staging block's worth of bytes and where on the device they go
  void* dev;
  size_t bytes;
};
using FillFn = std::function<bool(size_t job, char* blk)>;
using SentFn = std::function<hipError_t(size_t job, hipStream_t st)>;
static int copy_bytes_in(plr_ctx* c, const std::vector<CopyPiece>& pieces);
static int copy_rows_in(plr_ctx* c, int64_t row0, int64_t nrows, const double* X, int64_t ldx);

namespace {

using plr::FinishArgs;
using plr::PassArgs;

typedef void (*pass_fn)(PassArgs);

// The shapes and the width -> variant choice live in plr_plan.hpp (host-only,
// checked on a CPU for every width); here the kernel instances, in the same
// order.  [grad][allch]: rows handled by one wave and the tail-stage variants
// always match their variant exactly, so they carry only the allch instances.
using plr_plan::Shape;
using plr_plan::kShapes;
using plr_plan::kNumShapes;
using plr_plan::kBlkNch;
using plr_plan::kBlkWcol;
using plr_plan::kBlockCols;

struct VariantFns {
  pass_fn fn[2][2];
};

template <int NCH, int R, int WCOL, int WROW, int MINW, bool THL, int TL>
VariantFns make_fns() {
  VariantFns f = {{{nullptr, nullptr}, {nullptr, nullptr}}};
  f.fn[0][1] = plr::shard_pass<NCH, R, WCOL, WROW, MINW, false, true, THL, plr::kPassFused, TL>;
  f.fn[1][1] = plr::shard_pass<NCH, R, WCOL, WROW, MINW, true, true, THL, plr::kPassFused, TL>;
  if constexpr (WCOL > 1 && TL == 0) {
    f.fn[0][0] = plr::shard_pass<NCH, R, WCOL, WROW, MINW, false, false, THL>;
    f.fn[1][0] = plr::shard_pass<NCH, R, WCOL, WROW, MINW, true, false, THL>;
  }
  return f;
}

const VariantFns kFns[] = {
#define PLR_V(NCH, R, WCOL, WROW, MINW, THL, TL) make_fns<NCH, R, WCOL, WROW, MINW, THL, TL>(),
#include "plr_variants.def"
#undef PLR_V
};
static_assert(sizeof(kFns) / sizeof(kFns[0]) == (size_t)kNumShapes, "one kernel set per shape");

// Rows wider than the widest fused variant are processed in column blocks of
// 16384, in two sweeps over X (dot products of all blocks, then residuals,
// then the rank-1 updates of all blocks): X is read twice, but any width works.
// [allch]
const pass_fn kBlockDot[2] = {
    plr::shard_pass<kBlkNch, 1, kBlkWcol, 1, 2, false, false, true, plr::kPassDot>,
    plr::shard_pass<kBlkNch, 1, kBlkWcol, 1, 2, false, true, true, plr::kPassDot>};
const pass_fn kBlockAxpy[2] = {
    plr::shard_pass<kBlkNch, 1, kBlkWcol, 1, 2, true, false, true, plr::kPassAxpy>,
    plr::shard_pass<kBlkNch, 1, kBlkWcol, 1, 2, true, true, true, plr::kPassAxpy>};
// ... or, when the row fits a team of at most 16 workgroups, read once: each
// workgroup of a team owns one column block and the partial dot products are
// exchanged per row.  [grad]
typedef void (*team_fn)(plr::TeamArgs);
struct TeamFns {
  team_fn grad[2];  // team_pass: [identity link]
  team_fn dot;      // team_dot: the passes without a gradient
};
template <int NCH, int LAG>
TeamFns make_team_fns() {
  return {{plr::team_pass<NCH, false, LAG>, plr::team_pass<NCH, true, LAG>}, plr::team_dot<NCH>};
}
// [chunks per wave - kTeamMinNch][lag - 1]
const TeamFns kTeam[plr_plan::kTeamNch - plr_plan::kTeamMinNch + 1][2] = {
    {make_team_fns<7, 1>(), make_team_fns<7, 2>()},
    {make_team_fns<8, 1>(), make_team_fns<8, 2>()}};
static_assert(plr_plan::kTeamMinNch == 7 && plr_plan::kTeamNch == 8 &&
                  plr_plan::kTeamWaves == plr::kTeamWaves,
              "one team kernel set per chunk count");
constexpr int64_t kHostPredictCols = 192;  // from this pitch on predictions go straight to host
// Results watched for by the host thread (results_arrived): finishing kernels of
// up to 64 blocks (1024 columns), for at most 20 ms -- longer than any pass over
// a shard that fits the device -- before the thread waits for the stream instead.
constexpr int kDoneWords = 64;
constexpr int kPollLimitUs = 20000;
constexpr unsigned kTeamSpinLimit = 1u << 22;  // polls before a wait for a partner gives up

// Narrow rows (d <= 64): row-tiled layout, a lane per row.
struct LaneVariant {
  int np, U, wrow, wcol;  // wcol 2: a pair of waves shares every tile (lane2_pass)
  pass_fn fn[2];          // [grad]
};
#define PLR_LANE(NP, U, WROW, MINW)                       \
  {NP, U, WROW, 1,                                        \
   {plr::lane_pass<NP, U, WROW, MINW, false>, plr::lane_pass<NP, U, WROW, MINW, true>}}
#define PLR_LANE2(NP, U, MINW) \
  {NP, U, 1, 2, {plr::lane2_pass<NP, U, MINW, false>, plr::lane2_pass<NP, U, MINW, true>}}
// indexed by column pairs - 1; tiles per group, waves and register budget from
// sweeps over every combination on 1.6 GB shards (6.75-7.0 TB/s from 6
// columns up; 4 columns 5.9, 2 columns 4.2: one exp/log per 16-32 bytes).
// From 30 columns on a wave pair per tile is faster than a wave (+1-7 %).
const LaneVariant kLane[] = {
    PLR_LANE(1, 4, 4, 1),  // 2 columns
    PLR_LANE(2, 1, 8, 1),
    PLR_LANE(3, 2, 4, 2),
    PLR_LANE(4, 1, 8, 1),
    PLR_LANE(5, 1, 4, 1),
    PLR_LANE(6, 1, 4, 1),
    PLR_LANE(7, 1, 4, 1),
    PLR_LANE(8, 1, 4, 2),  // 16 columns
    PLR_LANE(9, 1, 4, 1),
    PLR_LANE(10, 1, 4, 2),
    PLR_LANE(11, 1, 4, 1),
    PLR_LANE(12, 1, 4, 1),
    PLR_LANE(13, 1, 4, 2),
    PLR_LANE(14, 1, 4, 1),
    PLR_LANE2(15, 2, 2),  // 30 columns
    PLR_LANE2(16, 2, 2),  // 32 columns
    PLR_LANE2(17, 2, 2),
    PLR_LANE2(18, 2, 2),
    PLR_LANE2(19, 2, 2),
    PLR_LANE2(20, 2, 2),
    PLR_LANE2(21, 2, 2),
    PLR_LANE2(22, 2, 2),
    PLR_LANE2(23, 2, 2),
    PLR_LANE2(24, 2, 2),
    PLR_LANE2(25, 1, 2),  // 50 columns
    PLR_LANE2(26, 1, 2),
    PLR_LANE2(27, 1, 2),
    PLR_LANE2(28, 1, 2),
    PLR_LANE2(29, 1, 2),
    PLR_LANE2(30, 1, 2),
    PLR_LANE2(31, 1, 2),
    PLR_LANE2(32, 1, 2),  // 64 columns
};
static_assert(sizeof(kLane) / sizeof(kLane[0]) == plr_plan::kMaxLaneCols / 2, "one variant per width");

// Rows of 65..96 columns: a half-wave per row, G row pairs per tile.
struct PairVariant {
  int G, wrow;
  pass_fn fn[2];  // [grad]
};
// 16 rows per tile, two waves per SIMD (sweeps on MI355X: 6.5-7.0 TB/s for
// every even pitch 66..96; taller tiles and other occupancies lose 5-20 %)
const PairVariant kPair = {8, 4, {plr::pair_pass<8, 4, 2, false>, plr::pair_pass<8, 4, 2, true>}};

// the column-blocked path's shape: 8 waves x 16 chunks, one row per tile, theta in LDS
const Shape kBlockShape = {kBlkNch, 1, kBlkWcol, 1, 2, true, 0};

std::string g_create_error;  // last failure of a call that has no context

// ---- static device scratch of plr_loss_grad_noalloc ------------------------
// Everything that entry point needs beyond the caller's inputs and outputs:
// the zero-padded copy of theta, the per-workgroup loss partials and the
// per-workgroup gradient partials.  One array per GPU, held until the process
// ends; every call on a GPU uses that GPU's copy.
constexpr int64_t kNaMaxPitch = 2048;  // widest row pitch (doubles) the entry point takes
constexpr int kNaMaxGrid = 512;        // most workgroups a pass may use
constexpr size_t kNaThetaOff = 0;
constexpr size_t kNaLossOff = kNaThetaOff + (size_t)kNaMaxPitch * sizeof(double);
constexpr size_t kNaPartOff = kNaLossOff + (size_t)kNaMaxGrid * sizeof(double);
constexpr size_t kNaScratchBytes =
    kNaPartOff + (size_t)kNaMaxGrid * kNaMaxPitch * sizeof(double);  // 8 MiB + 20 KiB
static_assert(kNaLossOff % 256 == 0 && kNaPartOff % 256 == 0, "sub-buffers stay aligned");

static __device__ __align__(256) unsigned char scratch[kNaScratchBytes];

// In host code `scratch` is only a handle for the symbol; the device address
// differs per GPU and is looked up once per device, with that device current.
constexpr int kNaMaxDevices = 64;
std::mutex g_na_mutex;
unsigned char* g_na_ptr[kNaMaxDevices] = {};
int g_na_num_cu[kNaMaxDevices] = {};
// workgroups per compute unit of the variant for a pitch of k chunks, per
// device (0: not asked yet): the occupancy query runs once per (device, pitch)
int g_na_occ[kNaMaxDevices][kNaMaxPitch / plr::kChunkCols + 1] = {};
std::mutex g_err_mutex;  // g_create_error is shared by every context-free call

}  // namespace

struct plr_ctx {
  int device = 0;
  int num_cu = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;

  // resident shard
  double* dX = nullptr;
  double* dy = nullptr;
  int64_t n = 0, d = 0, pitch = 0;
  bool have_data = false;
  // A first column that is 1.0 in every row (the bias column of the file path)
  // is not stored when the caller says so: the shard then holds dcols = d - 1
  // columns, theta's first entry lives in d_theta[bias_slot], and the sum of
  // the residuals (d_part_res) is that column's gradient.
  bool opt_first_col_one = false;  // plr_set_option("first_column_is_one")
  bool bias = false;               // in force for the resident shard
  int64_t dcols = 0;               // stored columns
  int64_t bias_slot = 0;
  double* d_part_res = nullptr;    // max(grid, grid_nograd)

  // per-shape workspace
  const Shape* var = nullptr;       // shape of the shard_pass variant in use
  const VariantFns* fns = nullptr;  // its kernel instances (fused path)
  int nch_rt = 0;
  int grid = 0, grid_nograd = 0;
  bool allch = false;
  int tail_cols = 0;            // columns handled by the variant's tail stage
  const LaneVariant* lane = nullptr;      // d <= 64: row-tiled layout, lane_pass
  int64_t n_alloc = 0;                    // rows the shard buffer holds (lane path: whole groups)
  double* up_dev = nullptr;               // lane path: device staging of uploaded row-major rows
  const PairVariant* pair = nullptr;      // 65..96 columns: half-wave rows
  bool blocked = false;         // rows wider than the widest fused variant: column blocks
  // ... read once by teams of workgroups (team_blocks > 0), else in two sweeps
  int team_blocks = 0, team_blk_chunks = 0, team_blk_extra = 0, team_nch = 0, nteams = 0;
  const TeamFns* team_fns = nullptr;
  int opt_team_lag = 0;      // plr_set_option("team_lag"): 0 = by shape
  int team_lag = 0;          // in force for the resident shard
  unsigned long long* d_zx = nullptr;  // [nteams][4][team_blocks][2] exchange slots, then the
                                       // status word of the pass
  int64_t zx_words = 0;
  unsigned team_spin_limit = kTeamSpinLimit;
  // A team pass needs its whole grid resident at once.  When it is not (other
  // processes or streams holding compute units) a workgroup gives up waiting,
  // and the pass is run again in two sweeps, which need no residency; after
  // kTeamGiveUpsAllowed such passes the shard stays on two sweeps.
  bool opt_team_fallback = true;  // plr_set_option("team_fallback")
  bool team_off = false;          // team passes switched off for the resident shard
  int team_giveups = 0;
  int sweep_grid = 0;             // grid of the two-sweep kernels (0: not sized yet)
  int64_t part_rows = 0;          // rows of pitch doubles that d_part_g holds
  int64_t part_len = 0;           // entries of d_part_loss and d_part_res
  std::string base_info;          // kernel description without the give-up note
  bool opt_two_sweeps = false;  // plr_set_option("column_blocks_two_sweeps")
  bool opt_csv_overlap = true;  // plr_set_option("csv_overlap")
  bool synth_first_col = false; // the shard being reserved comes from plr_set_data_csv
  int csv_slow_fields = 0;      // fields of the last plr_set_data_csv the host converted
  bool team_check = false;      // a team pass ran since the status word was last read
  double* d_z = nullptr;        // n: blocked rows only, x.theta accumulated over the blocks
  double* d_zparts = nullptr;   // [team_blocks * 8][n]: team_dot's partial dot products
  int64_t zstride = 0;          // entries per (wave, team) in d_zparts
  int res_grid = 1;             // workgroups of residual_pass behind a team pass
  double* d_res = nullptr;      // n: blocked rows only, residual per row
  int64_t theta_len = 0;
  double* d_theta = nullptr;    // theta_len doubles, zero padded
  double* d_part_g = nullptr;   // grid x pitch
  double* d_part_loss = nullptr;  // max(grid, grid_nograd)
  double* d_h = nullptr;        // n (predict), lazily allocated
  double* h_pred = nullptr;     // n, pinned + device-mapped: where wide shards put predictions
  double* h_pred_dev = nullptr;
  void* out_stage = nullptr;    // pinned staging of copy_rows_out, lazily allocated
  hipStream_t out_stream[8] = {};  // one per copy lane (kCopyLanes)
  double* d_curve = nullptr;    // per-round losses of plr_train_dgd, lazily allocated
  double* d_train_out = nullptr;  // d + 1: where training rounds put delta (never read back)
  int curve_len = 0;
  double* h_theta = nullptr;    // pinned + device-mapped, theta_len
  double* h_theta_dev = nullptr;  // the device's address of h_theta
  double* h_out = nullptr;      // pinned + device-mapped, d + 1: finish_pass writes it
  double* h_out_dev = nullptr;  // the device's address of h_out
  // behind h_out's d + 1 doubles, on a cache line of their own: the words the
  // finishing kernel's blocks store the pass number to (FinishArgs::done)
  volatile unsigned long long* h_done = nullptr;
  unsigned long long* h_done_dev = nullptr;
  volatile unsigned long long* h_status = nullptr;  // behind them: finish_pass's copy of a
  unsigned long long* h_status_dev = nullptr;       //   team pass's give-up word
  unsigned long long pass_seq = 0;
  int done_blocks = 0;          // > 0: the pass just enqueued reports through h_done
  bool opt_poll_results = true; // plr_set_option("poll_results")

  double last_ms = 0., sum_ms = 0.;
  int64_t launches = 0;
  bool timing = true;           // record the two events around the streaming kernels

  std::string err;
  std::string info;
};

namespace {

int fail(plr_ctx* c, int code, const std::string& msg) {
  if (c) c->err = msg;
  return code;
}

#define PLR_HIP(c, call)                                                     \
  do {                                                                       \
    hipError_t e_ = (call);                                                  \
    if (e_ != hipSuccess) {                                                  \
      char b_[512];                                                          \
      snprintf(b_, sizeof b_, "%s failed: %s (%s:%d)", #call,                \
               hipGetErrorString(e_), __FILE__, __LINE__);                   \
      (void)hipGetLastError();                                               \
      return fail((c), (e_ == hipErrorOutOfMemory) ? PLR_ERR_NOMEM           \
                                                   : PLR_ERR_HIP, b_);       \
    }                                                                        \
  } while (0)

void release_upload_staging(plr_ctx* c) {
  if (c->up_dev) (void)hipFree(c->up_dev);
  c->up_dev = nullptr;
}

void free_shape(plr_ctx* c) {
  (void)hipSetDevice(c->device);
  release_upload_staging(c);
  if (c->dX) (void)hipFree(c->dX);
  if (c->dy) (void)hipFree(c->dy);
  if (c->d_theta) (void)hipFree(c->d_theta);
  if (c->d_part_g) (void)hipFree(c->d_part_g);
  if (c->d_part_loss) (void)hipFree(c->d_part_loss);
  if (c->d_part_res) (void)hipFree(c->d_part_res);
  c->d_part_res = nullptr;
  c->bias = false;
  c->dcols = 0;
  if (c->d_h) (void)hipFree(c->d_h);
  if (c->h_pred) (void)hipHostFree(c->h_pred);
  c->h_pred = c->h_pred_dev = nullptr;
  if (c->d_curve) (void)hipFree(c->d_curve);
  if (c->d_zx) (void)hipFree(c->d_zx);
  c->d_zx = nullptr;
  c->team_blocks = c->team_blk_chunks = c->team_blk_extra = c->team_nch = c->nteams = 0;
  c->team_fns = nullptr;
  c->zx_words = 0;
  c->team_check = false;
  c->team_off = false;
  c->team_giveups = 0;
  c->sweep_grid = 0;
  c->part_rows = c->part_len = 0;
  c->base_info.clear();
  if (c->d_z) (void)hipFree(c->d_z);
  if (c->d_zparts) (void)hipFree(c->d_zparts);
  c->d_zparts = nullptr;
  if (c->d_res) (void)hipFree(c->d_res);
  if (c->d_train_out) (void)hipFree(c->d_train_out);
  if (c->h_theta) (void)hipHostFree(c->h_theta);
  if (c->h_out) (void)hipHostFree(c->h_out);
  c->dX = c->dy = c->d_theta = c->d_part_g = c->d_part_loss = c->d_h = c->d_curve = c->d_z = c->d_res =
      c->d_train_out = c->h_theta = c->h_theta_dev = c->h_out = c->h_out_dev = nullptr;
  c->n = c->d = c->pitch = 0;
  c->have_data = false;
  c->curve_len = 0;
  c->blocked = false;
  c->lane = nullptr;
  c->n_alloc = 0;
  c->pair = nullptr;
  c->tail_cols = 0;
  c->var = nullptr;
  c->fns = nullptr;
  c->info.clear();
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Grid of the two-sweep kernels of a column-blocked shard of n rows.
int size_sweep_grid(plr_ctx* c, int64_t n) {
  const int threads = plr::kWave * kBlkWcol;
  int occ = 0, occ2 = 0;
  PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                 &occ, reinterpret_cast<const void*>(kBlockAxpy[0]), threads, 0));
  PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                 &occ2, reinterpret_cast<const void*>(kBlockDot[0]), threads, 0));
  if (occ2 < occ) occ = occ2;
  if (occ < 1) return fail(c, PLR_ERR_HIP, "kernel variant does not fit on a compute unit");
  int64_t g = (int64_t)c->num_cu * occ;
  if (g > n) g = n;
  if (g < 1) g = 1;
  c->sweep_grid = (int)g;
  return PLR_OK;
}

// Pick the kernel variant (plr_plan.hpp) and the persistent grid for an
// n x d shard.
int plan_shape(plr_ctx* c, int64_t n, int64_t d) {
  plr_plan::Plan pl;
  if (!plr_plan::plan_width(d, pl, n))
    return fail(c, PLR_ERR_UNSUPPORTED, "no kernel variant covers this width");
  c->pitch = pl.pitch;
  c->theta_len = pl.theta_len;
  c->nch_rt = pl.nch_rt;
  c->allch = pl.allch;
  c->tail_cols = pl.tail_cols;
  if (pl.path == plr_plan::kPathLane) {
    const LaneVariant* lv = &kLane[pl.np - 1];
    const int threads = plr::kWave * lv->wrow * lv->wcol;
    c->lane = lv;
    c->var = &kBlockShape;  // unused by this path, kept non-null
    c->nch_rt = 1;
    int occ = 0, occ2 = 0;
    PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                   &occ, reinterpret_cast<const void*>(lv->fn[1]), threads, 0));
    PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                   &occ2, reinterpret_cast<const void*>(lv->fn[0]), threads, 0));
    if (occ < 1 || occ2 < 1)
      return fail(c, PLR_ERR_HIP, "kernel variant does not fit on a compute unit");
    const int64_t ngroups = ceil_div(n, (int64_t)plr::kWave * lv->U);
    const int64_t want = std::max<int64_t>(1, ceil_div(ngroups, lv->wrow));
    c->grid = (int)std::min<int64_t>(want, (int64_t)c->num_cu * occ);
    // (the instances without a gradient need fewer registers and would fit more
    // workgroups per compute unit; measured, they stream fastest on the grid of
    // the instance with one: more resident waves than the tile shape was tuned
    // for cost 1-6 %)
    c->grid_nograd = (int)std::min<int64_t>(want, (int64_t)c->num_cu * std::min(occ, occ2));
    char b[256];
    snprintf(b, sizeof b,
             "%s<NP=%d,U=%d,WROW=%d> row-tiled layout, pitch=%lld, %d rows per group, "
             "grid=%d x %d threads (occupancy %d blocks/CU, %d CUs)",
             lv->wcol == 2 ? "lane2_pass" : "lane_pass", lv->np, lv->U, lv->wrow, (long long)c->pitch, plr::kWave * lv->U, c->grid, threads,
             occ, c->num_cu);
    c->info = b;
    return PLR_OK;
  }
  if (pl.path == plr_plan::kPathPair) {
    const PairVariant* pv = &kPair;
    const int threads = plr::kWave * pv->wrow;
    c->pair = pv;
    c->var = &kBlockShape;  // unused by this path, kept non-null
    c->nch_rt = 1;
    int occ = 0, occ2 = 0;
    PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                   &occ, reinterpret_cast<const void*>(pv->fn[1]), threads, 0));
    PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                   &occ2, reinterpret_cast<const void*>(pv->fn[0]), threads, 0));
    if (occ < 1 || occ2 < 1)
      return fail(c, PLR_ERR_HIP, "kernel variant does not fit on a compute unit");
    const int64_t ntiles = ceil_div(n, (int64_t)2 * pv->G);
    const int64_t want = std::max<int64_t>(1, ceil_div(ntiles, pv->wrow));
    c->grid = (int)std::min<int64_t>(want, (int64_t)c->num_cu * occ);
    c->grid_nograd = (int)std::min<int64_t>(want, (int64_t)c->num_cu * std::min(occ, occ2));
    char b[256];
    snprintf(b, sizeof b,
             "pair_pass<G=%d,WROW=%d> pitch=%lld, %d rows per tile, grid=%d x %d threads "
             "(occupancy %d blocks/CU, %d CUs)",
             pv->G, pv->wrow, (long long)c->pitch, 2 * pv->G, c->grid, threads, occ, c->num_cu);
    c->info = b;
    return PLR_OK;
  }
  if (pl.path == plr_plan::kPathBlocked) {
    const int threads = plr::kWave * kBlkWcol;
    c->var = &kBlockShape;
    c->blocked = true;
    if (pl.team_blocks > 0 && !c->opt_two_sweeps) {
      // one read of X: teams of team_blocks workgroups, all resident at once.
      // Any of the instances may be launched on this shard, so the grid is
      // sized to the one that fits the fewest workgroups on a compute unit.
      const int lag = c->opt_team_lag ? c->opt_team_lag : pl.team_lag;
      const TeamFns* tf = &kTeam[pl.team_nch - plr_plan::kTeamMinNch][lag - 1];
      // (team_dot needs no residency; it runs on the same grid)
      int tocc = 1 << 30;
      for (int k = 0; k < 2; ++k) {
        int o = 0;
        PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                       &o, reinterpret_cast<const void*>(tf->grad[k]), threads, 0));
        if (o < tocc) tocc = o;
      }
      const int nteams = tocc * c->num_cu / pl.team_blocks;
      if (nteams >= 1) {
        c->team_fns = tf;
        c->team_blocks = pl.team_blocks;
        c->team_blk_chunks = pl.team_blk_chunks;
        c->team_blk_extra = pl.team_blk_extra;
        c->team_nch = pl.team_nch;
        c->team_lag = lag;
        c->nteams = nteams;
        c->grid = c->grid_nograd = c->nteams * c->team_blocks;
        c->zx_words = (int64_t)c->nteams * plr::kTeamSlots * c->team_blocks * 2;
        char b[256];
        snprintf(b, sizeof b,
                 "team_pass<NCH=%d,LAG=%d> %d column blocks of %d%s chunks, %d teams, pitch=%lld "
                 "grid=%d x %d threads (occupancy %d blocks/CU, %d CUs)",
                 c->team_nch, c->team_lag, c->team_blocks, c->team_blk_chunks,
                 c->team_blk_extra ? "-" : "", c->nteams, (long long)c->pitch, c->grid, threads,
                 tocc, c->num_cu);
        c->info = b;
        return PLR_OK;
      }
    }
    const int rc = size_sweep_grid(c, n);
    if (rc != PLR_OK) return rc;
    c->grid = c->grid_nograd = c->sweep_grid;
    char b[256];
    snprintf(b, sizeof b,
             "column-blocked shard_pass<NCH=%d,R=1,WCOL=%d> two sweeps over %lld blocks of %lld "
             "columns, pitch=%lld grid=%d x %d threads",
             kBlkNch, kBlkWcol, (long long)ceil_div(c->pitch, kBlockCols), (long long)kBlockCols,
             (long long)c->pitch, c->grid, threads);
    c->info = b;
    return PLR_OK;
  }
  const Shape* v = &kShapes[pl.variant];
  const VariantFns* f = &kFns[pl.variant];
  c->var = v;
  c->fns = f;
  if (!f->fn[1][c->allch] || !f->fn[0][c->allch])
    return fail(c, PLR_ERR_UNSUPPORTED, "kernel variant lacks the instance this width needs");
  const int threads = plr::kWave * v->wcol * v->wrow;
  const int64_t ntiles = ceil_div(n, v->R);
  const int64_t want = ceil_div(ntiles, v->wrow);
  int occ = 0, occ_ng = 0;
  PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                 &occ, reinterpret_cast<const void*>(f->fn[1][c->allch]), threads, 0));
  PLR_HIP(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(
                 &occ_ng, reinterpret_cast<const void*>(f->fn[0][c->allch]), threads, 0));
  if (occ < 1 || occ_ng < 1)
    return fail(c, PLR_ERR_HIP, "kernel variant does not fit on a compute unit");
  int64_t g = (int64_t)c->num_cu * occ, g2 = (int64_t)c->num_cu * std::min(occ, occ_ng);
  if (g > want) g = want;
  if (g2 > want) g2 = want;
  if (g < 1) g = 1;
  if (g2 < 1) g2 = 1;
  c->grid = (int)g;
  c->grid_nograd = (int)g2;
  char b[256];
  snprintf(b, sizeof b,
           "shard_pass<NCH=%d,R=%d,WCOL=%d,WROW=%d,ALLCH=%d,TL=%d> nch_rt=%d tail=%d pitch=%lld "
           "grid=%d x %d threads (occupancy %d blocks/CU, %d CUs)",
           v->nch, v->R, v->wcol, v->wrow, (int)c->allch, v->tl, c->nch_rt, c->tail_cols,
           (long long)c->pitch, c->grid, threads, occ, c->num_cu);
  c->info = b;
  return PLR_OK;
}

// The rows of an n x d shard: layout and kernel variant for that shape, then X
// (with the slack the kernels may read past the last row) and y.
int alloc_rows(plr_ctx* c, int64_t n, int64_t d, bool zero_fill) {
  c->bias = (c->opt_first_col_one || c->synth_first_col) && d >= 2;
  c->dcols = d - (c->bias ? 1 : 0);
  int rc = plan_shape(c, n, c->dcols);
  if (rc != PLR_OK) return rc;
  if (c->bias) c->info += "; first column constant 1, not stored";
  c->bias_slot = c->theta_len;  // behind the zero padding
  // sizes are computed in size_t below: a shard whose byte count does not fit
  // in 64 bits must be refused here, not wrap around to a small allocation
  // that the kernels would then stream far past
  const size_t slack_bytes = std::max<size_t>((size_t)c->theta_len * sizeof(double), 64u << 10);
  // the row-tiled layout holds whole groups of tiles; the rows past n are zeros
  const int64_t group_rows = c->lane ? (int64_t)plr::kWave * c->lane->U : 1;
  if (n > INT64_MAX - group_rows)
    return fail(c, PLR_ERR_INVALID, "n * pitch * 8 bytes does not fit in 64 bits");
  const int64_t n_alloc = ceil_div(n, group_rows) * group_rows;
  if ((uint64_t)n_alloc > (UINT64_MAX / sizeof(double) - slack_bytes) / (uint64_t)c->pitch)
    return fail(c, PLR_ERR_INVALID, "n * pitch * 8 bytes does not fit in 64 bits");
  c->n = n;
  c->n_alloc = n_alloc;
  c->d = d;
  // lanes of the chunk that straddles the end of the last row read (and then
  // discard) up to one slab past it: keep that much slack mapped
  const size_t xbytes = (size_t)n_alloc * c->pitch * sizeof(double) + slack_bytes;
  if (n > 0) {
    PLR_HIP(c, hipMalloc(&c->dX, xbytes));
    PLR_HIP(c, hipMalloc(&c->dy, (size_t)n * sizeof(double)));
    if (c->lane && !zero_fill) {
      // the last group of tiles: its rows past n are never uploaded
      const size_t last = (size_t)(n_alloc - group_rows) * c->pitch * sizeof(double);
      PLR_HIP(c, hipMemsetAsync(reinterpret_cast<char*>(c->dX) + last, 0, xbytes - last, c->stream));
    }
    if (zero_fill) {
      // a shard that is filled row range by row range: rows the caller never
      // sends must read as zeros, not as whatever the memory held
      PLR_HIP(c, hipMemsetAsync(c->dX, 0, xbytes, c->stream));
      PLR_HIP(c, hipMemsetAsync(c->dy, 0, (size_t)n * sizeof(double), c->stream));
    }
    if (c->pitch != c->dcols && !c->lane)  // the pad column must read as zero
      PLR_HIP(c, hipMemset2DAsync(c->dX + c->dcols, (size_t)c->pitch * sizeof(double), 0,
                                  (size_t)(c->pitch - c->dcols) * sizeof(double), (size_t)n,
                                  c->stream));
  }
  return PLR_OK;
}

// Everything else a pass over the resident rows needs: theta and result
// staging, the per-workgroup partials of the variant chosen for (c->n, c->d).
int alloc_workspace(plr_ctx* c) {
  const int64_t n = c->n, d = c->d;
  const int gmax = c->grid > c->grid_nograd ? c->grid : c->grid_nograd;
  PLR_HIP(c, hipMalloc(&c->d_theta, (size_t)(c->theta_len + 8) * sizeof(double)));
  // a team shares one row of gradient partials
  c->part_rows = c->team_blocks > 0 ? c->nteams : c->grid;
  // behind a team pass residual_pass folds the row terms: a thread per row
  c->res_grid = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(n, 256), 2 * c->num_cu));
  c->part_len = std::max(gmax, c->res_grid);
  PLR_HIP(c, hipMalloc(&c->d_part_res, (size_t)c->part_len * sizeof(double)));
  PLR_HIP(c, hipMalloc(&c->d_part_g, (size_t)c->part_rows * c->pitch * sizeof(double)));
  PLR_HIP(c, hipMalloc(&c->d_part_loss, (size_t)c->part_len * sizeof(double)));
  if (c->team_blocks > 0) {
    // exchange slots, then the status word; the slots are cleared before every
    // launch, the status word only here and when the host has read a give-up
    PLR_HIP(c, hipMalloc(&c->d_zx, (size_t)(c->zx_words + 1) * sizeof(unsigned long long)));
    PLR_HIP(c, hipMemsetAsync(c->d_zx, 0, (size_t)(c->zx_words + 1) * sizeof(unsigned long long),
                              c->stream));
    // z per row (team_pass), and every wave's partial of it (team_dot)
    PLR_HIP(c, hipMalloc(&c->d_z, (size_t)std::max<int64_t>(n, 1) * sizeof(double)));
    c->zstride = ceil_div(ceil_div(std::max<int64_t>(n, 1), c->nteams), plr::kWave) * plr::kWave;
    PLR_HIP(c, hipMalloc(&c->d_zparts, (size_t)c->zstride * c->nteams * c->team_blocks *
                                           plr::kTeamWaves * sizeof(double)));
  } else if (c->blocked && n > 0) {
    PLR_HIP(c, hipMalloc(&c->d_z, (size_t)n * sizeof(double)));
    PLR_HIP(c, hipMalloc(&c->d_res, (size_t)n * sizeof(double)));
  }
  PLR_HIP(c, hipHostMalloc(&c->h_theta, (size_t)(c->theta_len + 8) * sizeof(double),
                           hipHostMallocMapped | hipHostMallocCoherent));
  PLR_HIP(c, hipHostGetDevicePointer(reinterpret_cast<void**>(&c->h_theta_dev), c->h_theta, 0));
  // results land in host memory straight from the finishing kernel (no
  // device-to-host copy in the step): pinned, mapped, coherent
  const size_t done_at = ((size_t)(d + 1) + 7) / 8 * 8;  // in doubles: the next cache line
  PLR_HIP(c, hipHostMalloc(&c->h_out, (done_at + kDoneWords + 8) * sizeof(double),
                           hipHostMallocMapped | hipHostMallocCoherent));
  PLR_HIP(c, hipHostGetDevicePointer(reinterpret_cast<void**>(&c->h_out_dev), c->h_out, 0));
  memset(c->h_out, 0, (done_at + kDoneWords + 8) * sizeof(double));
  c->h_done = reinterpret_cast<volatile unsigned long long*>(c->h_out + done_at);
  c->h_done_dev = reinterpret_cast<unsigned long long*>(c->h_out_dev + done_at);
  c->h_status = c->h_done + kDoneWords;
  c->h_status_dev = c->h_done_dev + kDoneWords;
  memset(c->h_theta, 0, (size_t)(c->theta_len + 8) * sizeof(double));
  PLR_HIP(c, hipMemsetAsync(c->d_theta, 0, (size_t)(c->theta_len + 8) * sizeof(double), c->stream));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  c->base_info = c->info;
  c->have_data = true;
  return PLR_OK;
}

int alloc_shape_buffers(plr_ctx* c, int64_t n, int64_t d, bool zero_fill) {
  const int rc = alloc_rows(c, n, d, zero_fill);
  return rc != PLR_OK ? rc : alloc_workspace(c);
}

// Drop the resident shard (if any) and reserve an n x d one.  On failure the
// context is left without a shard (shape 0 x 0), never half allocated.
int alloc_shape(plr_ctx* c, int64_t n, int64_t d, bool zero_fill) {
  if (n < 0 || d < 1)
    return fail(c, PLR_ERR_INVALID, "need n >= 0 and d >= 1");
  PLR_HIP(c, hipSetDevice(c->device));
  free_shape(c);
  const int rc = alloc_shape_buffers(c, n, d, zero_fill);
  if (rc != PLR_OK) free_shape(c);  // keeps c->err
  return rc;
}

int upload_rows(plr_ctx* c, int64_t row0, int64_t nrows, const double* X,
                int64_t ldx, const double* y) {
  if (nrows == 0) return PLR_OK;
  if (!X || !y) return fail(c, PLR_ERR_INVALID, "X and y must not be NULL");
  if (ldx < c->d) return fail(c, PLR_ERR_INVALID, "ldx must be >= d");
  if (row0 < 0 || nrows < 0 || row0 + nrows > c->n)
    return fail(c, PLR_ERR_INVALID, "row range outside the reserved shard");
  PLR_HIP(c, hipSetDevice(c->device));
  const int rc = copy_rows_in(c, row0, nrows, X, ldx);
  if (rc != PLR_OK) return rc;
  return copy_bytes_in(c, {{c->dy + row0, y, (size_t)nrows * sizeof(double)}});
}

enum PassKind { kPassGrad, kPassDelta, kPassLoss, kPassPredict, kPassPredictLinear };

// Enqueue one pass on the context's stream: streaming kernel (between the two
// timing events) and finishing kernel.  theta must already be in d_theta.
// `out` receives d values + the loss; train_round >= 0 makes the finishing
// kernel also apply delta to the device theta and store the loss in
// d_curve[train_round].
int enqueue_pass(plr_ctx* c, PassKind kind, unsigned loss_mode, double alpha, double beta,
                 double* out, int train_round) {
  const Shape* v = c->var;
  const bool grad = (kind == kPassGrad || kind == kPassDelta);
  const bool predict = (kind == kPassPredict || kind == kPassPredictLinear);
  c->done_blocks = 0;
  // rows shared by a team of workgroups: with a gradient the one-read pass with
  // its exchange (unless switched off), without one the exchange-free team_dot
  const bool team = c->team_blocks > 0 && !c->team_off && grad;
  const bool team_dot = c->team_blocks > 0 && !grad;
  const int grid = (c->blocked && !team && !team_dot) ? c->sweep_grid
                   : grad                             ? c->grid
                                                      : c->grid_nograd;
  const int threads = c->lane ? plr::kWave * c->lane->wrow * c->lane->wcol
                      : c->pair ? plr::kWave * c->pair->wrow
                                : plr::kWave * v->wcol * v->wrow;

  PassArgs pa;
  pa.X = c->dX;
  pa.y = predict ? nullptr : c->dy;
  pa.theta = c->d_theta;
  pa.part_g = c->d_part_g;
  pa.part_loss = c->d_part_loss;
  pa.h_out = predict ? (c->h_pred_dev ? c->h_pred_dev : c->d_h) : nullptr;
  pa.n = c->n;
  pa.pitch = c->pitch;
  pa.ntiles = ceil_div(c->n, v->R);
  pa.nch_rt = c->nch_rt;
  pa.tail_cols = c->tail_cols;
  pa.loss_mode = predict ? (unsigned)plr::kLossNone : loss_mode;
  pa.identity_link = (kind == kPassPredictLinear || loss_mode == plr::kLossSquared) ? 1 : 0;

  pa.theta_bias = c->bias ? c->d_theta + c->bias_slot : nullptr;
  pa.part_res = c->bias ? c->d_part_res : nullptr;
  pa.width = c->pitch;
  pa.z_buf = nullptr;
  pa.z_accumulate = 0;
  pa.res_in = nullptr;

  if (c->timing) PLR_HIP(c, hipEventRecord(c->ev0, c->stream));
  if (c->lane) {
    hipLaunchKernelGGL(c->lane->fn[grad ? 1 : 0], dim3(grid), dim3(threads), 0, c->stream, pa);
    PLR_HIP(c, hipGetLastError());
  } else if (c->pair) {
    hipLaunchKernelGGL(c->pair->fn[grad ? 1 : 0], dim3(grid), dim3(threads), 0, c->stream, pa);
    PLR_HIP(c, hipGetLastError());
  } else if (!c->blocked) {
    hipLaunchKernelGGL(c->fns->fn[grad ? 1 : 0][c->allch ? 1 : 0], dim3(grid), dim3(threads), 0,
                       c->stream, pa);
    PLR_HIP(c, hipGetLastError());
  } else if (team || team_dot) {
    plr::TeamArgs ta;
    ta.X = c->dX;
    ta.y = pa.y;
    ta.theta = c->d_theta;
    ta.part_g = c->d_part_g;
    ta.n = c->n;
    ta.pitch = c->pitch;
    ta.nblk = c->team_blocks;
    ta.nteams = c->nteams;
    ta.blk_chunks = c->team_blk_chunks;
    ta.blk_extra = c->team_blk_extra;
    ta.theta_bias = pa.theta_bias;
    ta.zeros = c->d_theta + c->theta_len - plr::kChunkCols;  // the padding never changes
    ta.zx = c->d_zx;
    ta.status = reinterpret_cast<unsigned*>(c->d_zx + c->zx_words);
    ta.spin_limit = c->team_spin_limit;
    int zparts = 0;
    if (grad) {
      // the exchange slots start at zero (sequence number 0 = empty).  The status
      // word behind them is NOT cleared here: a give-up in any pass of a chain of
      // passes enqueued back to back must still be there when the host looks.
      hipLaunchKernelGGL(plr::fill_zero, dim3(16), dim3(256), 0, c->stream,
                         reinterpret_cast<double*>(c->d_zx), c->zx_words);
      PLR_HIP(c, hipGetLastError());
      ta.z_out = c->d_z;
      ta.zstride = 0;
      hipLaunchKernelGGL(c->team_fns->grad[pa.identity_link], dim3(c->grid), dim3(threads), 0,
                         c->stream, ta);
      PLR_HIP(c, hipGetLastError());
      c->team_check = true;
    } else {
      // no gradient: every wave's partial dot products, no exchange
      ta.z_out = c->d_zparts;
      ta.zstride = c->zstride;
      zparts = c->team_blocks;
      hipLaunchKernelGGL(c->team_fns->dot, dim3(c->grid), dim3(threads), 0, c->stream, ta);
      PLR_HIP(c, hipGetLastError());
    }
    // z -> loss terms, predictions, sum of the residuals
    hipLaunchKernelGGL(plr::residual_pass, dim3(c->res_grid), dim3(256), 0, c->stream,
                       (const double*)ta.z_out, (const double*)pa.y, (double*)nullptr, pa.h_out,
                       c->d_part_loss, c->n, pa.loss_mode, pa.identity_link, pa.theta_bias,
                       pa.part_res, zparts, c->nteams, c->zstride);
    PLR_HIP(c, hipGetLastError());
  } else if (c->n > 0) {
    // sweep 1: z = x.theta, one launch per column block, accumulated in d_z
    pa.z_buf = c->d_z;
    double* const pred_out = pa.h_out;  // the residual kernel writes the predictions
    pa.h_out = nullptr;
    for (int64_t col0 = 0; col0 < c->pitch; col0 += kBlockCols) {
      const int64_t w = std::min<int64_t>(kBlockCols, c->pitch - col0);
      PassArgs pb = pa;
      pb.X = c->dX + col0;
      pb.theta = c->d_theta + col0;
      pb.width = w;
      pb.nch_rt = (int)ceil_div(ceil_div(w, plr::kChunkCols), kBlkWcol);
      pb.z_accumulate = col0 > 0 ? 1 : 0;
      hipLaunchKernelGGL(kBlockDot[w == kBlockCols ? 1 : 0], dim3(grid), dim3(threads), 0,
                         c->stream, pb);
      PLR_HIP(c, hipGetLastError());
    }
    // residual, prediction and loss per row
    hipLaunchKernelGGL(plr::residual_pass, dim3(grid), dim3(256), 0, c->stream,
                       (const double*)c->d_z, (const double*)pa.y, grad ? c->d_res : nullptr,
                       pred_out, c->d_part_loss, c->n, pa.loss_mode,
                       pa.identity_link, pa.theta_bias, pa.part_res, 0, 0, (int64_t)0);
    PLR_HIP(c, hipGetLastError());
    // sweep 2: rank-1 updates, block by block
    if (grad) {
      pa.res_in = c->d_res;
      for (int64_t col0 = 0; col0 < c->pitch; col0 += kBlockCols) {
        const int64_t w = std::min<int64_t>(kBlockCols, c->pitch - col0);
        PassArgs pb = pa;
        pb.X = c->dX + col0;
        pb.theta = c->d_theta + col0;
        pb.part_g = c->d_part_g + col0;
        pb.width = w;
        pb.nch_rt = (int)ceil_div(ceil_div(w, plr::kChunkCols), kBlkWcol);
        hipLaunchKernelGGL(kBlockAxpy[w == kBlockCols ? 1 : 0], dim3(grid), dim3(threads), 0,
                           c->stream, pb);
        PLR_HIP(c, hipGetLastError());
      }
    }
  } else {
    // empty shard: the finishing kernel needs zeroed partials
    PLR_HIP(c, hipMemsetAsync(c->d_part_loss, 0, (size_t)grid * sizeof(double), c->stream));
    PLR_HIP(c, hipMemsetAsync(c->d_part_res, 0, (size_t)grid * sizeof(double), c->stream));
    if (grad)
      PLR_HIP(c, hipMemsetAsync(c->d_part_g, 0, (size_t)grid * c->pitch * sizeof(double),
                                c->stream));
  }
  if (c->timing) PLR_HIP(c, hipEventRecord(c->ev1, c->stream));

  if (!predict) {
    FinishArgs fa;
    fa.part_g = c->d_part_g;
    fa.part_loss = c->d_part_loss;
    fa.theta = c->d_theta;
    fa.out = out;
    fa.pitch = c->pitch;
    fa.d = c->dcols;
    fa.n = c->n;
    fa.part_res = pa.part_res;
    fa.theta_bias = c->d_theta + c->bias_slot;
    fa.nparts = team ? c->nteams : grid;  // a team shares one row of partials
    fa.nparts_loss = (team || team_dot) ? c->res_grid : grid;
    fa.delta_mode = (kind == kPassDelta) ? (train_round >= 0 ? 2 : 1) : 0;
    fa.have_grad = grad ? 1 : 0;
    const int fblocks = grad ? (int)ceil_div(c->dcols, plr::kFinCols) : 1;
    // a pass short enough for the stream's own completion signal to matter
    // reports to the polling host thread as well (run_pass)
    fa.status_in = team ? reinterpret_cast<const unsigned*>(c->d_zx + c->zx_words) : nullptr;
    fa.status_out = c->h_status_dev;
    fa.done = nullptr;
    fa.seq = 0;
    if (c->opt_poll_results && out == c->h_out_dev && fblocks <= kDoneWords) {
      c->done_blocks = fblocks;
      fa.done = c->h_done_dev;
      fa.seq = ++c->pass_seq;
    }
    fa.alpha = alpha;
    fa.coff2 = 2. * beta * alpha;
    fa.theta_rw = c->d_theta;
    fa.loss_slot = (train_round >= 0 && c->d_curve) ? c->d_curve + train_round : nullptr;
    const int fgrid = grad ? (int)ceil_div(c->dcols, plr::kFinCols) : 1;
    hipLaunchKernelGGL(plr::finish_pass, dim3(fgrid),
                       dim3(plr::kFinCols * plr::kFinSlices), 0, c->stream, fa);
    PLR_HIP(c, hipGetLastError());
  }
  return PLR_OK;
}

// theta (host) -> pinned staging -> device copy, by a kernel on the stream
int stage_theta_from_host(plr_ctx* c, const double* theta) {
  memcpy(c->h_theta, theta, (size_t)c->d * sizeof(double));
  const int sgrid = (int)((c->d + 1023) / 1024 > 64 ? 64 : (c->d + 1023) / 1024);
  hipLaunchKernelGGL(plr::stage_theta, dim3(sgrid), dim3(256), 0, c->stream,
                     (const double*)c->h_theta_dev, c->d_theta, c->d, c->bias ? 1 : 0,
                     c->bias_slot);
  PLR_HIP(c, hipGetLastError());
  return PLR_OK;
}

int account_timing(plr_ctx* c) {
  if (!c->timing) return PLR_OK;
  float ms = 0.f;
  hipError_t e = hipEventElapsedTime(&ms, c->ev0, c->ev1);
  if (e == hipErrorNotReady) {  // (the results were polled for: the stream may trail them)
    (void)hipGetLastError();
    PLR_HIP(c, hipEventSynchronize(c->ev1));
    e = hipEventElapsedTime(&ms, c->ev0, c->ev1);
  }
  PLR_HIP(c, e);
  c->last_ms = ms;
  c->sum_ms += ms;
  c->launches += 1;
  return PLR_OK;
}

// After the stream has drained: did a workgroup of a team pass give up waiting
// for a partner?  Then the results of every pass since the last look are not
// the shard's.  Returns 1 if so (the status word is cleared again), 0 if not,
// a negative status if the look itself failed.
int team_gave_up(plr_ctx* c) {
  if (!c->team_check) return 0;
  c->team_check = false;
  // (the finishing kernel of every team pass leaves a copy of the word in host memory)
  if ((unsigned)*c->h_status == 0u) return 0;
  *c->h_status = 0;
  PLR_HIP(c, hipMemset(c->d_zx + c->zx_words, 0, sizeof(unsigned long long)));
  return 1;
}

constexpr int kTeamGiveUpsAllowed = 2;  // then the shard stays on two sweeps

// A team pass gave up.  Either report it (fallback switched off), or make the
// two-sweep path ready -- its grid, z and residual vectors, partials for its
// grid -- and switch the team path off: for the pass that is run again right
// away (the caller switches it back on afterwards unless this was the last
// give-up allowed), or for good.
int fall_back_to_two_sweeps(plr_ctx* c) {
  if (!c->opt_team_fallback)
    return fail(c, PLR_ERR_HIP,
                "team pass: a workgroup gave up waiting for its partners' partial dot products "
                "(are all workgroups of the grid resident?); results discarded");
  c->team_giveups += 1;
  if (c->sweep_grid == 0) {
    const int rc = size_sweep_grid(c, c->n);
    if (rc != PLR_OK) return rc;
  }
  if (!c->d_res && c->n > 0)  // (d_z exists: the team pass stores z there too)
    PLR_HIP(c, hipMalloc(&c->d_res, (size_t)c->n * sizeof(double)));
  if (c->part_rows < c->sweep_grid) {
    PLR_HIP(c, hipFree(c->d_part_g));
    c->d_part_g = nullptr;
    c->part_rows = 0;
    PLR_HIP(c, hipMalloc(&c->d_part_g, (size_t)c->sweep_grid * c->pitch * sizeof(double)));
    c->part_rows = c->sweep_grid;
  }
  if (c->part_len < c->sweep_grid) {
    PLR_HIP(c, hipFree(c->d_part_loss));
    PLR_HIP(c, hipFree(c->d_part_res));
    c->d_part_loss = c->d_part_res = nullptr;
    c->part_len = 0;
    PLR_HIP(c, hipMalloc(&c->d_part_loss, (size_t)c->sweep_grid * sizeof(double)));
    PLR_HIP(c, hipMalloc(&c->d_part_res, (size_t)c->sweep_grid * sizeof(double)));
    c->part_len = c->sweep_grid;
  }
  c->team_off = true;
  char b[200];
  snprintf(b, sizeof b, "; %d team pass%s gave up waiting and ran again in two sweeps%s",
           c->team_giveups, c->team_giveups == 1 ? "" : "es",
           c->team_giveups >= kTeamGiveUpsAllowed ? ", team passes now off for this shard" : "");
  c->info = c->base_info + b;
  return PLR_OK;
}

// A short pass's results are in host memory microseconds before the runtime
// reports the stream drained: the finishing kernel's blocks store the pass
// number behind the results, and this thread watches those words.  False when
// the pass does not report that way or the words have not all arrived within
// the time limit (the caller then waits for the stream, which also brings a
// kernel's failure to light).  The stream may still be finishing the kernel's
// last instructions when this returns true; later work is ordered behind it.
bool results_arrived(plr_ctx* c) {
  const int nb = c->done_blocks;
  if (nb <= 0) return false;
  const unsigned long long seq = c->pass_seq;
  const auto t0 = std::chrono::steady_clock::now();
  for (unsigned spin = 1;; ++spin) {
    int b = 0;
    while (b < nb && c->h_done[b] == seq) ++b;
    if (b == nb) {
      std::atomic_thread_fence(std::memory_order_acquire);
      return true;
    }
    if ((spin & 255u) == 0 &&
        std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(kPollLimitUs))
      return false;
    __builtin_ia32_pause();
  }
}

// One synchronous pass: theta in, kernels, results in the mapped host buffer.
int run_pass(plr_ctx* c, PassKind kind, const double* theta, unsigned loss_mode,
             double alpha, double beta) {
  if (!c->have_data) return fail(c, PLR_ERR_NODATA, "no shard resident: call plr_set_data first");
  if (!theta) return fail(c, PLR_ERR_INVALID, "theta must not be NULL");
  if (loss_mode > plr::kLossSquared) return fail(c, PLR_ERR_INVALID, "unknown loss flag");
  PLR_HIP(c, hipSetDevice(c->device));
  const bool predict = (kind == kPassPredict || kind == kPassPredictLinear);
  if (predict && !c->d_h && !c->h_pred && c->n > 0) {
    // Where the predictions go.  A row of kHostPredictCols columns or more
    // streams slowly enough (8 bytes out per >= 1.5 KiB in) for the host link
    // to keep up: the kernel then writes straight into pinned host memory --
    // no HBM write traffic disturbing the read stream, no copy command
    // afterwards.  Narrower rows produce predictions faster than the link
    // takes them; they go to device memory and are copied out in a pipeline.
    if (c->pitch >= kHostPredictCols) {
      PLR_HIP(c, hipHostMalloc(&c->h_pred, (size_t)c->n * sizeof(double),
                               hipHostMallocMapped | hipHostMallocCoherent));
      PLR_HIP(c, hipHostGetDevicePointer(reinterpret_cast<void**>(&c->h_pred_dev), c->h_pred, 0));
    } else {
      PLR_HIP(c, hipMalloc(&c->d_h, (size_t)c->n * sizeof(double)));
    }
  }
  int rc = stage_theta_from_host(c, theta);
  if (rc != PLR_OK) return rc;
  rc = enqueue_pass(c, kind, loss_mode, alpha, beta, c->h_out_dev, -1);
  if (rc != PLR_OK) return rc;
  // (measured: hipStreamSynchronize returns ~7 us sooner than a hipStreamQuery poll loop)
  if (!results_arrived(c)) PLR_HIP(c, hipStreamSynchronize(c->stream));
  rc = team_gave_up(c);
  if (rc < 0) return rc;
  if (rc == 1) {
    // theta is still staged; the same pass once more, in two sweeps
    rc = fall_back_to_two_sweeps(c);
    if (rc != PLR_OK) return rc;
    rc = enqueue_pass(c, kind, loss_mode, alpha, beta, c->h_out_dev, -1);
    if (rc != PLR_OK) return rc;
    PLR_HIP(c, hipStreamSynchronize(c->stream));
    if (c->team_giveups < kTeamGiveUpsAllowed) c->team_off = false;
  }
  return account_timing(c);
}

}  // namespace

extern "C" {

int plr_create(plr_ctx** out, int device_id) {
  auto set_err = [](const std::string& m) {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    g_create_error = m;
  };
  if (!out) {
    set_err("out must not be NULL");
    return PLR_ERR_INVALID;
  }
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count < 1) {
    (void)hipGetLastError();
    set_err(std::string("no HIP device available: ") + hipGetErrorString(e));
    return PLR_ERR_HIP;
  }
  if (device_id < 0 || device_id >= count) {
    set_err("device_id out of range");
    return PLR_ERR_INVALID;
  }
  plr_ctx* c = new plr_ctx();
  c->device = device_id;
  hipDeviceProp_t prop;
  if ((e = hipSetDevice(device_id)) != hipSuccess ||
      (e = hipGetDeviceProperties(&prop, device_id)) != hipSuccess ||
      (e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking)) != hipSuccess ||
      (e = hipEventCreate(&c->ev0)) != hipSuccess ||
      (e = hipEventCreate(&c->ev1)) != hipSuccess) {
    set_err(std::string("context set-up failed: ") + hipGetErrorString(e));
    (void)hipGetLastError();
    plr_destroy(c);
    return PLR_ERR_HIP;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_err(std::string("device is ") + prop.gcnArchName +
            "; this library carries gfx950 code only");
    plr_destroy(c);
    return PLR_ERR_UNSUPPORTED;
  }
  c->num_cu = prop.multiProcessorCount;
  *out = c;
  return PLR_OK;
}

void plr_destroy(plr_ctx* c) {
  if (!c) return;
  free_shape(c);
  if (c->out_stage) (void)hipHostFree(c->out_stage);
  for (hipStream_t st : c->out_stream)
    if (st) (void)hipStreamDestroy(st);
  if (c->ev0) (void)hipEventDestroy(c->ev0);
  if (c->ev1) (void)hipEventDestroy(c->ev1);
  if (c->stream) (void)hipStreamDestroy(c->stream);
  delete c;
}

int plr_alloc_data(plr_ctx* c, int64_t n, int64_t d) {
  if (!c) return PLR_ERR_INVALID;
  return alloc_shape(c, n, d, /*zero_fill=*/true);
}

int plr_set_data_chunk(plr_ctx* c, int64_t row0, int64_t nrows, const double* X,
                       int64_t ldx, const double* y) {
  if (!c) return PLR_ERR_INVALID;
  if (!c->have_data) return fail(c, PLR_ERR_NODATA, "call plr_alloc_data first");
  return upload_rows(c, row0, nrows, X, ldx, y);
}

int plr_set_data(plr_ctx* c, const double* X, int64_t n, int64_t d, int64_t ldx,
                 const double* y) {
  if (!c) return PLR_ERR_INVALID;
  if (n > 0 && (!X || !y)) return fail(c, PLR_ERR_INVALID, "X and y must not be NULL");
  if (ldx < d) return fail(c, PLR_ERR_INVALID, "ldx must be >= d");
  int rc = alloc_shape(c, n, d, /*zero_fill=*/false);  // every row is uploaded right below
  if (rc != PLR_OK) return rc;
  rc = upload_rows(c, 0, n, X, ldx, y);
  if (rc != PLR_OK) {
    // a shard that was not filled (a refused first column, a failed copy) must
    // not stay resident: later passes would run on whatever the memory holds
    const std::string why = c->err;
    free_shape(c);
    c->err = why;
  }
  return rc;
}

// ---------------------------------------------------------------------------
// plr_set_data_csv: the worker's share of the sample text, parsed on the device

namespace {

struct DevBuf {  // device memory released on every exit path
  void* p = nullptr;
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
};

struct ShardGuard {  // a shard that was not completed does not stay resident
  plr_ctx* c;
  bool done = false;
  ~ShardGuard() {
    if (!done) free_shape(c);
  }
};

// fields of the first non-empty line (maximal runs of non-separator bytes)
int64_t first_line_fields(const char* const* text, const int64_t* len, int nspans, char sep) {
  for (int s = 0; s < nspans; ++s) {
    const char* t = text[s];
    int64_t i = 0;
    while (i < len[s] && t[i] == '\n') ++i;
    if (i == len[s]) continue;
    int64_t fields = 0;
    bool in_field = false;
    for (; i < len[s] && t[i] != '\n'; ++i) {
      if (t[i] == sep) {
        in_field = false;
      } else if (!in_field) {
        in_field = true;
        ++fields;
      }
    }
    return fields;
  }
  return 0;
}

}  // namespace

static int copy_rows_out(plr_ctx* c, double* out, const double* dev, size_t count);

// The sample text as it lies on the device: the spans back to back, a newline
// behind each (it keeps their lines apart), then kCsvPadBytes of newlines.
struct CsvText {
  const char* const* text;
  const int64_t* len;
  int nspans;
  int64_t total = 0;             // bytes with the newline behind every span
  int64_t padded = 0;            // bytes of the device buffer
  std::vector<int64_t> span_at;  // device offset of every span
};

// Fields the device left to the host (longer digit strings, inf, nan, hex, ...):
// std::stod on the host's copy of the text, then patched into the shard.
static int resolve_slow_fields(plr_ctx* c, const CsvText& ct, int64_t d, char sep, int nslow,
                               const void* d_slow) {
  if (nslow <= 0) return PLR_OK;
  std::vector<plr::CsvSlow> slow(nslow);
  PLR_HIP(c, hipMemcpy(slow.data(), d_slow, (size_t)nslow * sizeof(plr::CsvSlow),
                       hipMemcpyDeviceToHost));
  std::vector<int64_t> xi, yi;
  std::vector<double> xv, yv;
  for (const plr::CsvSlow& f : slow) {
    int s = 0;
    while (s + 1 < ct.nspans && f.pos >= ct.span_at[s + 1]) ++s;
    const char* p = ct.text[s] + (f.pos - ct.span_at[s]);
    const char* const end = ct.text[s] + ct.len[s];
    int64_t flen = f.len;
    if (flen < 0) {
      flen = 0;
      while (p + flen < end && p[flen] != sep && p[flen] != '\n') ++flen;
    }
    double v;
    try {
      v = std::stod(std::string(p, (size_t)flen));
    } catch (const std::exception& e) {  // what the reference's parser would have thrown
      return fail(c, PLR_ERR_INVALID, std::string(e.what()) + ": field " + std::to_string(f.col) +
                                          " of sample line " + std::to_string(f.row));
    }
    if (f.col == d - 1) {
      yi.push_back(f.row);
      yv.push_back(v);
    } else if (c->lane) {
      const int64_t np = c->lane->np;
      xi.push_back(((((f.row >> 6) * np + (f.col >> 1)) << 6) + (f.row & 63)) * 2 + (f.col & 1));
      xv.push_back(v);
    } else {
      xi.push_back(f.row * c->pitch + f.col);
      xv.push_back(v);
    }
  }
  auto patch = [&](double* base, const std::vector<int64_t>& idx,
                   const std::vector<double>& val) -> int {
    if (idx.empty()) return PLR_OK;
    DevBuf di, dv;
    PLR_HIP(c, hipMalloc(&di.p, idx.size() * sizeof(int64_t)));
    PLR_HIP(c, hipMalloc(&dv.p, val.size() * sizeof(double)));
    PLR_HIP(c, hipMemcpy(di.p, idx.data(), idx.size() * sizeof(int64_t), hipMemcpyHostToDevice));
    PLR_HIP(c, hipMemcpy(dv.p, val.data(), val.size() * sizeof(double), hipMemcpyHostToDevice));
    hipLaunchKernelGGL(plr::csv_patch, dim3((unsigned)((idx.size() + 255) / 256)), dim3(256), 0,
                       c->stream, base, static_cast<const int64_t*>(di.p),
                       static_cast<const double*>(dv.p), (int64_t)idx.size());
    PLR_HIP(c, hipGetLastError());
    PLR_HIP(c, hipStreamSynchronize(c->stream));
    return PLR_OK;
  };
  int rc = patch(c->dX, xi, xv);
  if (rc == PLR_OK) rc = patch(c->dy, yi, yv);
  return rc;
}

constexpr int kCsvSlowCap = 1 << 20;
constexpr int kCsvRetrySerial = 1;  // the pipelined parse leaves the input to the serial one

// What both parses end with: the parser's verdict, the fields left to the
// host, the description.
static int finish_csv(plr_ctx* c, const CsvText& ct, int64_t d, char sep, const int64_t res[3],
                      const void* d_slow, const char* parser, const char* how = "") {
  if (res[1] != INT64_MAX)  // parse_lines' message for the same input
    return fail(c, PLR_ERR_INVALID, "ragged sample line " + std::to_string(res[1]));
  if (res[2] > (int64_t)kCsvSlowCap)
    return fail(c, PLR_ERR_UNSUPPORTED,
                "more than 2^20 fields need the host's number parser: parse this input there");
  const int nslow = (int)res[2];
  const int rc = resolve_slow_fields(c, ct, d, sep, nslow, d_slow);
  if (rc != PLR_OK) return rc;
  c->csv_slow_fields = nslow;
  c->info += std::string("; parsed from text") + how + " (" + parser + "), " +
             std::to_string(nslow) + " fields converted on the host";
  c->base_info = c->info;
  if (c->timing) {  // plr_get_timing's last_ms: the parsing kernel(s)
    float ms = 0.f;
    PLR_HIP(c, hipEventElapsedTime(&ms, c->ev0, c->ev1));
    c->last_ms = ms;
  }
  return PLR_OK;
}

static plr::CsvFieldArgs csv_field_args(plr_ctx* c, const unsigned char* dt,
                                        const int64_t* first_row, const int64_t* first_field,
                                        int64_t rows_cap, int64_t d, char sep, plr::CsvSlow* slow,
                                        int64_t* ctl) {
  plr::CsvFieldArgs fa;
  fa.text = dt;
  fa.first_row = first_row;
  fa.first_field = first_field;
  fa.block0 = 0;
  fa.rows_cap = rows_cap;
  fa.d = (int)d;
  fa.sep = (unsigned char)sep;
  fa.inv_d = 1.0 / (double)d;
  fa.X = c->dX;
  fa.y = c->dy;
  fa.pitch = c->pitch;
  fa.np = c->lane ? c->lane->np : 0;
  fa.slow = slow;
  fa.slow_cap = kCsvSlowCap;
  fa.slow_count = reinterpret_cast<unsigned long long*>(ctl + 2);
  fa.bad_row = reinterpret_cast<long long*>(ctl + 1);
  return fa;
}

// Transfer, then parse: the whole text goes to the device, the rows are counted
// (the host learns n and reserves exactly that shard), then located and parsed.
static int csv_serial(plr_ctx* c, const CsvText& ct, int64_t d, char sep, int64_t* n_out) {
  DevBuf d_text, d_slow, d_ctl;
  const int64_t total = ct.total;
  if (hipMalloc(&d_text.p, (size_t)ct.padded) != hipSuccess) {
    (void)hipGetLastError();
    return fail(c, PLR_ERR_NOMEM, "cannot allocate the device copy of the sample text");
  }
  unsigned char* dt = static_cast<unsigned char*>(d_text.p);
  std::vector<CopyPiece> pieces;
  for (int s = 0; s < ct.nspans; ++s) {
    if (ct.len[s]) pieces.push_back({dt + ct.span_at[s], ct.text[s], (size_t)ct.len[s]});
    PLR_HIP(c, hipMemsetAsync(dt + ct.span_at[s] + ct.len[s], '\n', 1, c->stream));
  }
  {
    const int rc = copy_bytes_in(c, pieces);
    if (rc != PLR_OK) return rc;
  }
  PLR_HIP(c, hipMemsetAsync(dt + total, '\n', (size_t)(ct.padded - total), c->stream));

  const int64_t nblocks = (total + plr::kCsvBlockBytes - 1) / plr::kCsvBlockBytes;
  if (nblocks > (int64_t)INT32_MAX) return fail(c, PLR_ERR_INVALID, "sample text too large");

  // rows and fields per block, and what lies in front of every block
  DevBuf d_rcount, d_fcount, d_frow, d_ffield;
  PLR_HIP(c, hipMalloc(&d_rcount.p, (size_t)nblocks * sizeof(int)));
  PLR_HIP(c, hipMalloc(&d_fcount.p, (size_t)nblocks * sizeof(int)));
  PLR_HIP(c, hipMalloc(&d_frow.p, (size_t)nblocks * sizeof(int64_t)));
  PLR_HIP(c, hipMalloc(&d_ffield.p, (size_t)nblocks * sizeof(int64_t)));
  PLR_HIP(c, hipMalloc(&d_ctl.p, 4 * sizeof(int64_t)));  // rows, bad row, slow fields, fields
  int64_t* ctl = static_cast<int64_t*>(d_ctl.p);
  const int64_t ctl_init[4] = {0, INT64_MAX, 0, 0};
  PLR_HIP(c, hipMemcpyAsync(ctl, ctl_init, sizeof ctl_init, hipMemcpyHostToDevice, c->stream));
  hipLaunchKernelGGL(plr::csv_count_blocks, dim3((unsigned)nblocks), dim3(plr::kCsvThreads), 0,
                     c->stream, dt, (unsigned char)sep, static_cast<int*>(d_rcount.p),
                     static_cast<int*>(d_fcount.p), (int64_t)0);
  hipLaunchKernelGGL(plr::csv_scan_blocks, dim3(1), dim3(1024), 0, c->stream,
                     static_cast<const int*>(d_rcount.p), static_cast<const int*>(d_fcount.p),
                     nblocks, static_cast<int64_t*>(d_frow.p), static_cast<int64_t*>(d_ffield.p),
                     ctl);
  PLR_HIP(c, hipGetLastError());
  int64_t tot[4] = {0, 0, 0, 0};
  PLR_HIP(c, hipMemcpyAsync(tot, ctl, sizeof tot, hipMemcpyDeviceToHost, c->stream));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  const int64_t n = tot[0], nfields = tot[3];
  if (n_out) *n_out = n;

  // the shard: k = d - 1 feature columns; the sample's constant first column is
  // not stored.  Every field of every row is written by the parser (a line with
  // another number of fields fails the call), so only the padding is cleared.
  c->synth_first_col = true;
  int rc = alloc_shape_buffers(c, n, d, /*zero_fill=*/false);
  c->synth_first_col = false;
  if (rc != PLR_OK) return rc;
  PLR_HIP(c, hipMalloc(&d_slow.p, (size_t)kCsvSlowCap * sizeof(plr::CsvSlow)));
  plr::CsvFieldArgs fa = csv_field_args(c, dt, static_cast<const int64_t*>(d_frow.p),
                                        static_cast<const int64_t*>(d_ffield.p), n, d, sep,
                                        static_cast<plr::CsvSlow*>(d_slow.p), ctl);
  if (c->timing) PLR_HIP(c, hipEventRecord(c->ev0, c->stream));
  hipLaunchKernelGGL(plr::csv_parse_fields, dim3((unsigned)nblocks), dim3(plr::kCsvThreads), 0,
                     c->stream, fa);
  PLR_HIP(c, hipGetLastError());
  if (c->timing) PLR_HIP(c, hipEventRecord(c->ev1, c->stream));
  int64_t res[4] = {0, 0, 0, 0};
  PLR_HIP(c, hipMemcpyAsync(res, ctl, sizeof res, hipMemcpyDeviceToHost, c->stream));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  // the line-start checks cover every row but the last
  if (res[1] == INT64_MAX && nfields != n * d) res[1] = n - 1;
  return finish_csv(c, ct, d, sep, res, d_slow.p, "a lane per field");
}

// Lines per byte from a sample of the text: the lengths of up to 256 lines at
// evenly spaced places.  0 when no line was found.
static double sampled_line_bytes(const CsvText& ct) {
  double sum = 0.;
  int64_t cnt = 0;
  const int kSamples = 4096;  // lines whose lengths vary by half their mean: +-0.8 %
  for (int i = 0; i < kSamples; ++i) {
    const int64_t off = (int64_t)((double)ct.total * i / kSamples);
    int s = 0;
    while (s + 1 < ct.nspans && off >= ct.span_at[s + 1]) ++s;
    const char* t = ct.text[s];
    const int64_t L = ct.len[s];
    int64_t p = std::min<int64_t>(off - ct.span_at[s], L);
    if (i > 0 || p > 0) {  // the line in progress at `off` is skipped
      const void* nl = p < L ? memchr(t + p, '\n', (size_t)(L - p)) : nullptr;
      if (!nl) continue;
      p = static_cast<const char*>(nl) - t + 1;
    }
    while (p < L && t[p] == '\n') ++p;  // empty lines are no rows
    if (p >= L) continue;
    const void* e = memchr(t + p, '\n', (size_t)(L - p));
    const int64_t end = e ? static_cast<const char*>(e) - t : L;
    sum += (double)(end - p + 1);
    ++cnt;
  }
  return cnt ? sum / (double)cnt : 0.;
}

struct LaneProgress;
static int lanes_in(plr_ctx* c, const std::vector<InJob>& jobs, const FillFn& fill,
                    const SentFn& sent, const char* what, LaneProgress* prog,
                    const std::function<int()>* conductor);

// Parse while the text arrives.  The text crosses the host link in 4 MiB blocks
// on the copy lanes; cut into stretches (64 MiB, the last one 16 MiB), every
// stretch is counted, scanned and parsed on the context's stream as soon as it
// and the 64 bytes behind it are on the device -- so the parser works in the
// shadow of the transfer and only the last stretch's kernels are left when the
// last byte has arrived.  The per-block parser does not care how few rows a
// stretch holds: a stretch of 16 MiB is 4096 workgroups.
// The shard has to exist before the number of rows is known: it is reserved
// for an estimate from the lengths of 4096 sampled lines plus 1/32 and 4096 rows;
// the few rows reserved in excess stay allocated.  Whenever that does not work
// out -- more rows than reserved, no memory for the generous shard -- the call
// falls back to csv_serial (kCsvRetrySerial; nothing is left behind).
// plr_set_option("csv_overlap", 0) switches it off.  Measured on 1.96 GB of
// text (rows of 512 six-decimal fields), the two alternating in one process,
// 12 calls each: median 39.0 ms against 45.3 ms for transfer-then-parse (the
// count and the parse, 5.7 ms, gone from the critical path).  The transfer
// itself is a little slower beside the kernels than alone: the copy lanes'
// streams and the kernels' stream share the device's few hardware queues, and
// a block queued behind a kernel waits for it.
constexpr int64_t kCsvStretch = 64ll << 20, kCsvLastStretch = 16ll << 20;
static_assert(kCsvLastStretch % (int64_t)kCopyBlock == 0 &&
                  (int64_t)kCopyBlock % plr::kCsvBlockBytes == 0,
              "a stretch is whole copy blocks and whole counting blocks");

struct LaneProgress {
  std::vector<hipEvent_t> done;            // per job: recorded behind its transfer
  std::atomic<size_t> issued[kCopyLanes];  // jobs lane l has issued (its k-th job is l + 8 k)
  std::atomic<bool> failed{false};
  ~LaneProgress() {
    for (hipEvent_t e : done)
      if (e) (void)hipEventDestroy(e);
  }
};

static int csv_pipelined(plr_ctx* c, const CsvText& ct, int64_t d, char sep, int64_t* n_out) {
  const int64_t total = ct.total;
  const double line_bytes = sampled_line_bytes(ct);
  if (line_bytes <= 0.) return kCsvRetrySerial;
  const int64_t n_est = (int64_t)((double)total / line_bytes);
  const int64_t cap = n_est + n_est / 32 + 4096;
  const int64_t nblocks = ceil_div(total, (int64_t)plr::kCsvBlockBytes);
  if (nblocks > (int64_t)INT32_MAX) return kCsvRetrySerial;
  // stretch boundaries (multiples of the copy block, so of the counting block)
  std::vector<int64_t> bound(1, 0);
  {
    const int64_t last = (total - kCsvLastStretch) / (int64_t)kCopyBlock * (int64_t)kCopyBlock;
    for (int64_t b = kCsvStretch; b + kCsvStretch / 2 < last; b += kCsvStretch) bound.push_back(b);
    if (last > bound.back()) bound.push_back(last);
    bound.push_back(total);
  }
  const int64_t nslabs = (int64_t)bound.size() - 1;
  DevBuf d_text, d_rcount, d_fcount, d_frow, d_ffield, d_slow, d_ctl;
  if (hipMalloc(&d_text.p, (size_t)ct.padded) != hipSuccess) {
    (void)hipGetLastError();
    return kCsvRetrySerial;
  }
  unsigned char* dt = static_cast<unsigned char*>(d_text.p);
  for (int s = 0; s < ct.nspans; ++s)
    PLR_HIP(c, hipMemsetAsync(dt + ct.span_at[s] + ct.len[s], '\n', 1, c->stream));
  PLR_HIP(c, hipMemsetAsync(dt + total, '\n', (size_t)(ct.padded - total), c->stream));

  // the transfer's jobs, in text order
  std::vector<InJob> jobs;
  std::vector<const char*> src;
  std::vector<int64_t> job_end;  // device offset behind every job
  for (int s = 0; s < ct.nspans; ++s)
    for (int64_t at = 0; at < ct.len[s]; at += (int64_t)kCopyBlock) {
      const size_t m = (size_t)std::min<int64_t>((int64_t)kCopyBlock, ct.len[s] - at);
      jobs.push_back({dt + ct.span_at[s] + at, m});
      src.push_back(ct.text[s] + at);
      job_end.push_back(ct.span_at[s] + at + (int64_t)m);
    }
  LaneProgress prog;
  prog.done.assign(jobs.size(), nullptr);
  for (size_t j = 0; j < jobs.size(); ++j)
    PLR_HIP(c, hipEventCreateWithFlags(&prog.done[j], hipEventDisableTiming));
  for (int l = 0; l < kCopyLanes; ++l) prog.issued[l].store(0);

  int64_t res[4] = {0, INT64_MAX, 0, 0};
  int fallback = 0;  // set by the conductor: leave the input to csv_serial
  const std::function<int()> conductor = [&]() -> int {
    // (runs on the calling thread while the lanes move the text)
    c->synth_first_col = true;
    int rc = alloc_rows(c, cap, d, /*zero_fill=*/false);
    c->synth_first_col = false;
    if (rc == PLR_ERR_NOMEM) {
      fallback = 1;
      return PLR_OK;
    }
    if (rc != PLR_OK) return rc;
    if (hipMalloc(&d_rcount.p, (size_t)nblocks * sizeof(int)) != hipSuccess ||
        hipMalloc(&d_fcount.p, (size_t)nblocks * sizeof(int)) != hipSuccess ||
        hipMalloc(&d_frow.p, (size_t)nblocks * sizeof(int64_t)) != hipSuccess ||
        hipMalloc(&d_ffield.p, (size_t)nblocks * sizeof(int64_t)) != hipSuccess ||
        hipMalloc(&d_slow.p, (size_t)kCsvSlowCap * sizeof(plr::CsvSlow)) != hipSuccess ||
        hipMalloc(&d_ctl.p, 4 * sizeof(int64_t)) != hipSuccess) {
      (void)hipGetLastError();
      fallback = 1;
      return PLR_OK;
    }
    int64_t* ctl = static_cast<int64_t*>(d_ctl.p);  // rows so far, bad row, slow fields, fields so far
    const int64_t ctl_init[4] = {0, INT64_MAX, 0, 0};
    PLR_HIP(c, hipMemcpyAsync(ctl, ctl_init, sizeof ctl_init, hipMemcpyHostToDevice, c->stream));
    plr::CsvFieldArgs fa = csv_field_args(c, dt, static_cast<const int64_t*>(d_frow.p),
                                          static_cast<const int64_t*>(d_ffield.p), cap, d, sep,
                                          static_cast<plr::CsvSlow*>(d_slow.p), ctl);
    size_t ready = 0;  // jobs [0, ready) are behind the context's stream already
    for (int64_t s = 0; s < nslabs; ++s) {
      // what this stretch needs on the device: itself and what a field that starts at its
      // end may still read
      const int64_t need = std::min<int64_t>(total, bound[s + 1] + plr::kCsvPadBytes);
      size_t upto = ready;
      while (upto < jobs.size() && job_end[upto] - (int64_t)jobs[upto].bytes < need) ++upto;
      for (int l = 0; l < kCopyLanes; ++l) {
        // lane l's jobs below `upto`: l, l + 8, ...
        const size_t mine = upto > (size_t)l ? (upto - l + kCopyLanes - 1) / kCopyLanes : 0;
        while (prog.issued[l].load(std::memory_order_acquire) < mine) {
          if (prog.failed.load()) return PLR_OK;  // the lanes report the error
          std::this_thread::sleep_for(std::chrono::microseconds(20));
        }
        if (mine > 0 && (size_t)l + (mine - 1) * kCopyLanes >= ready)
          PLR_HIP(c, hipStreamWaitEvent(c->stream, prog.done[l + (mine - 1) * kCopyLanes], 0));
      }
      ready = upto;
      const int64_t b0 = bound[s] / plr::kCsvBlockBytes;
      const int64_t nb = ceil_div(bound[s + 1], (int64_t)plr::kCsvBlockBytes) - b0;
      if (s == 0 && c->timing) PLR_HIP(c, hipEventRecord(c->ev0, c->stream));
      hipLaunchKernelGGL(plr::csv_count_blocks, dim3((unsigned)nb), dim3(plr::kCsvThreads), 0,
                         c->stream, dt, (unsigned char)sep, static_cast<int*>(d_rcount.p),
                         static_cast<int*>(d_fcount.p), b0);
      hipLaunchKernelGGL(plr::csv_scan_blocks, dim3(1), dim3(1024), 0, c->stream,
                         static_cast<const int*>(d_rcount.p) + b0,
                         static_cast<const int*>(d_fcount.p) + b0, nb,
                         static_cast<int64_t*>(d_frow.p) + b0,
                         static_cast<int64_t*>(d_ffield.p) + b0, ctl);
      fa.block0 = b0;
      hipLaunchKernelGGL(plr::csv_parse_fields, dim3((unsigned)nb), dim3(plr::kCsvThreads), 0,
                         c->stream, fa);
      PLR_HIP(c, hipGetLastError());
    }
    if (c->timing) PLR_HIP(c, hipEventRecord(c->ev1, c->stream));
    PLR_HIP(c, hipMemcpyAsync(res, ctl, sizeof res, hipMemcpyDeviceToHost, c->stream));
    return PLR_OK;
  };
  int rc = lanes_in(
      c, jobs,
      [&](size_t j, char* blk) {
        memcpy(blk, src[j], jobs[j].bytes);
        return true;
      },
      SentFn(), "copying the sample text to the device failed", &prog, &conductor);
  if (rc != PLR_OK) return rc;
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  if (fallback || res[0] > cap) return kCsvRetrySerial;

  // the exact shape: n rows of the cap reserved; variant, grid and workspace for n
  const int64_t n = res[0];
  if (n_out) *n_out = n;
  if (res[1] == INT64_MAX && res[3] != n * d) res[1] = n - 1;  // the last row's field count
  if (c->lane && n < c->n_alloc) {
    // the row-tiled layout's last group: its rows past n must read as zeros
    const int64_t group = (int64_t)plr::kWave * c->lane->U;
    const int64_t hi = std::min(c->n_alloc, ceil_div(std::max<int64_t>(n, 1), group) * group);
    if (hi > n) {
      hipLaunchKernelGGL(plr::zero_tiled_rows, dim3((unsigned)ceil_div((hi - n) * c->lane->np, 256)),
                         dim3(256), 0, c->stream, c->dX, c->lane->np, n, hi);
      PLR_HIP(c, hipGetLastError());
    }
  }
  c->n = n;
  rc = plan_shape(c, n, c->dcols);
  if (rc != PLR_OK) return rc;
  if (c->bias) c->info += "; first column constant 1, not stored";
  c->bias_slot = c->theta_len;
  rc = alloc_workspace(c);
  if (rc != PLR_OK) return rc;
  return finish_csv(c, ct, d, sep, res, d_slow.p, "a lane per field", " while it arrived");
}

int plr_set_data_csv(plr_ctx* c, const char* const* text, const int64_t* len, int nspans,
                     char sep, int64_t* n_out, int64_t* d_out) {
  if (!c) return PLR_ERR_INVALID;
  if (nspans < 0 || (nspans > 0 && (!text || !len)))
    return fail(c, PLR_ERR_INVALID, "text and len must not be NULL");
  if (sep == '\n' || sep == '\0') return fail(c, PLR_ERR_INVALID, "bad separator");
  CsvText ct;
  ct.text = text;
  ct.len = len;
  ct.nspans = nspans;
  ct.span_at.assign(nspans + 1, 0);
  for (int s = 0; s < nspans; ++s) {
    if (len[s] < 0 || (len[s] > 0 && !text[s]))
      return fail(c, PLR_ERR_INVALID, "bad text span");
    ct.span_at[s + 1] = ct.span_at[s] + len[s] + 1;  // a newline behind every span
  }
  ct.total = ct.span_at[nspans];
  // (whole counting blocks, then the pad the parsers may read ahead into)
  ct.padded = ceil_div(ct.total, (int64_t)plr::kCsvBlockBytes) * plr::kCsvBlockBytes +
              plr::kCsvPadBytes;
  const int64_t d = first_line_fields(text, len, nspans, sep);
  if (n_out) *n_out = 0;
  if (d_out) *d_out = d;
  if (d == 0) {  // no sample line at all: an empty shard
    PLR_HIP(c, hipSetDevice(c->device));
    free_shape(c);
    return PLR_OK;
  }
  if (d < 2)
    return fail(c, PLR_ERR_UNSUPPORTED, "lines of one field (a label and no feature) are not "
                                        "parsed on the device");
  if (d > (int64_t)INT32_MAX) return fail(c, PLR_ERR_INVALID, "too many fields in a line");
  PLR_HIP(c, hipSetDevice(c->device));
  free_shape(c);
  if (c->opt_csv_overlap && ct.total >= 4 * kCsvStretch) {
    ShardGuard guard{c};
    const int rc = csv_pipelined(c, ct, d, sep, n_out);
    if (rc == PLR_OK) guard.done = true;
    if (rc != kCsvRetrySerial) return rc;
  }
  ShardGuard guard{c};
  const int rc = csv_serial(c, ct, d, sep, n_out);
  if (rc == PLR_OK) guard.done = true;
  return rc;
}

int plr_get_data(plr_ctx* c, int64_t row0, int64_t nrows, double* X, int64_t ldx, double* y) {
  if (!c) return PLR_ERR_INVALID;
  if (!c->have_data) return fail(c, PLR_ERR_NODATA, "no shard resident: call plr_set_data first");
  if (row0 < 0 || nrows < 0 || row0 + nrows > c->n)
    return fail(c, PLR_ERR_INVALID, "row range outside the resident shard");
  if (nrows == 0) return PLR_OK;
  if (!X && !y) return fail(c, PLR_ERR_INVALID, "X and y must not both be NULL");
  if (X && ldx < c->d) return fail(c, PLR_ERR_INVALID, "ldx must be >= d");
  PLR_HIP(c, hipSetDevice(c->device));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  if (X) {
    // blocks of rows are brought to the caller's form on the device (dense rows of d
    // doubles, the constant column included), then copied out through the pinned lanes
    const int64_t d = c->d;
    const int64_t chunk_rows = std::max<int64_t>(1, (int64_t)(256u << 20) / (d * 8));
    DevBuf stage;
    PLR_HIP(c, hipMalloc(&stage.p, (size_t)std::min(chunk_rows, nrows) * d * sizeof(double)));
    for (int64_t r0 = 0; r0 < nrows; r0 += chunk_rows) {
      const int64_t m = std::min(chunk_rows, nrows - r0);
      hipLaunchKernelGGL(plr::gather_rows, dim3((unsigned)ceil_div(m * d, 256)), dim3(256), 0,
                         c->stream, (const double*)c->dX, c->pitch, c->lane ? c->lane->np : 0,
                         row0 + r0, m, (int)d, c->bias ? 1 : 0, static_cast<double*>(stage.p));
      PLR_HIP(c, hipGetLastError());
      PLR_HIP(c, hipStreamSynchronize(c->stream));
      if (ldx == d) {
        const int rc = copy_rows_out(c, X + r0 * ldx, static_cast<const double*>(stage.p),
                                     (size_t)(m * d));
        if (rc != PLR_OK) return rc;
      } else {
        PLR_HIP(c, hipMemcpy2D(X + r0 * ldx, (size_t)ldx * sizeof(double), stage.p,
                               (size_t)d * sizeof(double), (size_t)d * sizeof(double), (size_t)m,
                               hipMemcpyDeviceToHost));
      }
    }
  }
  if (y) {
    const int rc = copy_rows_out(c, y, c->dy + row0, (size_t)nrows);
    if (rc != PLR_OK) return rc;
  }
  return PLR_OK;
}

int plr_loss_grad(plr_ctx* c, const double* theta, double* gsum, double* loss_sum,
                  int64_t* n_out, unsigned flags) {
  if (!c) return PLR_ERR_INVALID;
  int rc = run_pass(c, kPassGrad, theta, flags, 0., 0.);
  if (rc != PLR_OK) return rc;
  if (gsum) memcpy(gsum, c->h_out, (size_t)c->d * sizeof(double));
  if (loss_sum) *loss_sum = c->h_out[c->d];
  if (n_out) *n_out = c->n;
  return PLR_OK;
}

int plr_dgd_delta(plr_ctx* c, const double* theta, double alpha, double beta,
                  double* delta, double* loss_sum) {
  if (!c) return PLR_ERR_INVALID;
  if (!delta) return fail(c, PLR_ERR_INVALID, "delta must not be NULL");
  int rc = run_pass(c, kPassDelta, theta,
                    loss_sum ? plr::kLossReference : plr::kLossNone, alpha, beta);
  if (rc != PLR_OK) return rc;
  memcpy(delta, c->h_out, (size_t)c->d * sizeof(double));
  if (loss_sum) *loss_sum = c->h_out[c->d];
  return PLR_OK;
}

int plr_dgd_delta_linear(plr_ctx* c, const double* theta, double alpha, double beta,
                         double* delta, double* loss_sum) {
  if (!c) return PLR_ERR_INVALID;
  if (!delta) return fail(c, PLR_ERR_INVALID, "delta must not be NULL");
  // the squared-loss formula selects the identity link; its loss term costs
  // one multiply per row, so it is always evaluated
  int rc = run_pass(c, kPassDelta, theta, plr::kLossSquared, alpha, beta);
  if (rc != PLR_OK) return rc;
  memcpy(delta, c->h_out, (size_t)c->d * sizeof(double));
  if (loss_sum) *loss_sum = c->h_out[c->d];
  return PLR_OK;
}

int plr_train_dgd(plr_ctx* c, double* theta, double alpha, double beta, int rounds,
                  double* loss_curve) {
  if (!c) return PLR_ERR_INVALID;
  if (!c->have_data) return fail(c, PLR_ERR_NODATA, "no shard resident: call plr_set_data first");
  if (!theta || rounds < 0) return fail(c, PLR_ERR_INVALID, "need theta and rounds >= 0");
  if (rounds == 0) return PLR_OK;
  PLR_HIP(c, hipSetDevice(c->device));
  if (c->curve_len < rounds) {
    if (c->d_curve) PLR_HIP(c, hipFree(c->d_curve));
    c->d_curve = nullptr;
    PLR_HIP(c, hipMalloc(&c->d_curve, (size_t)rounds * sizeof(double)));
    c->curve_len = rounds;
  }
  if (!c->d_train_out)
    PLR_HIP(c, hipMalloc(&c->d_train_out, (size_t)(c->d + 1) * sizeof(double)));
  const unsigned loss_mode = loss_curve ? plr::kLossReference : plr::kLossNone;
  const int skip = c->bias ? 1 : 0;
  int rc = PLR_OK;
  for (int attempt = 0;; ++attempt) {
    rc = stage_theta_from_host(c, theta);
    if (rc != PLR_OK) return rc;
    // every round is enqueued back to back; theta never leaves the device
    for (int rd = 0; rd < rounds; ++rd) {
      rc = enqueue_pass(c, kPassDelta, loss_mode, alpha, beta, c->d_train_out, rd);
      if (rc != PLR_OK) return rc;
    }
    PLR_HIP(c, hipMemcpyAsync(c->h_theta + skip, c->d_theta, (size_t)c->dcols * sizeof(double),
                              hipMemcpyDeviceToHost, c->stream));
    if (c->bias)
      PLR_HIP(c, hipMemcpyAsync(c->h_theta, c->d_theta + c->bias_slot, sizeof(double),
                                hipMemcpyDeviceToHost, c->stream));
    PLR_HIP(c, hipStreamSynchronize(c->stream));
    // a give-up in ANY round leaves the status word set (it is not cleared
    // between rounds) and every later round ran on a theta that is not the
    // shard's: the whole training is run again from the caller's theta, in two
    // sweeps
    rc = team_gave_up(c);
    if (rc < 0) return rc;
    if (rc == 0) break;
    rc = fall_back_to_two_sweeps(c);
    if (rc != PLR_OK) return rc;
    if (attempt >= 1) return fail(c, PLR_ERR_HIP, "team pass gave up although switched off");
  }
  if (c->team_off && c->team_giveups < kTeamGiveUpsAllowed) c->team_off = false;
  memcpy(theta, c->h_theta, (size_t)c->d * sizeof(double));
  if (loss_curve)
    PLR_HIP(c, hipMemcpy(loss_curve, c->d_curve, (size_t)rounds * sizeof(double),
                         hipMemcpyDeviceToHost));
  // the timing events were re-recorded every round: only the last round's pair is meaningful
  rc = account_timing(c);
  return rc;
}

int plr_calc_loss(plr_ctx* c, const double* theta, double* loss_sum, int64_t* n_out,
                  unsigned flags) {
  if (!c) return PLR_ERR_INVALID;
  if (flags == PLR_LOSS_NONE) return fail(c, PLR_ERR_INVALID, "plr_calc_loss needs a loss formula");
  int rc = run_pass(c, kPassLoss, theta, flags, 0., 0.);
  if (rc != PLR_OK) return rc;
  if (loss_sum) *loss_sum = c->h_out[c->d];
  if (n_out) *n_out = c->n;
  return PLR_OK;
}

// n doubles from the device into the caller's (pageable) buffer.  One plain
// copy command moves them through the runtime's own staging at ~10 GB/s; for
// tall shards that is several times the kernel.  Large results therefore go
// through kCopyLanes independent lanes, each with two pinned staging blocks on
// a stream of its own: the DMA into one block overlaps the host copy out of
// the other, and the lanes overlap each other.
static_assert(sizeof(plr_ctx::out_stream) / sizeof(hipStream_t) == kCopyLanes,
              "one stream per copy lane");

// pinned host memory -> the caller's buffer, kCopyLanes threads
static void copy_host_parallel(double* out, const double* src, size_t count) {
  if (count * sizeof(double) < (8u << 20)) {
    memcpy(out, src, count * sizeof(double));
    return;
  }
  std::thread th[kCopyLanes];
  const size_t per = (count + kCopyLanes - 1) / kCopyLanes;
  for (int l = 0; l < kCopyLanes; ++l)
    th[l] = std::thread([=]() {
      const size_t lo = std::min(count, (size_t)l * per), hi = std::min(count, lo + per);
      if (hi > lo) memcpy(out + lo, src + lo, (hi - lo) * sizeof(double));
    });
  for (int l = 0; l < kCopyLanes; ++l) th[l].join();
}

static int copy_rows_out(plr_ctx* c, double* out, const double* dev, size_t count) {
  const size_t bytes = count * sizeof(double);
  if (bytes < 4 * kCopyBlock) {
    PLR_HIP(c, hipMemcpy(out, dev, bytes, hipMemcpyDeviceToHost));
    return PLR_OK;
  }
  if (!c->out_stage) {
    PLR_HIP(c, hipHostMalloc(&c->out_stage, 2 * kCopyLanes * kCopyBlock, hipHostMallocDefault));
    for (int l = 0; l < kCopyLanes; ++l)
      PLR_HIP(c, hipStreamCreateWithFlags(&c->out_stream[l], hipStreamNonBlocking));
  }
  hipError_t errs[kCopyLanes];
  std::thread th[kCopyLanes];
  const size_t per_lane = ((count + kCopyLanes - 1) / kCopyLanes + 511) & ~(size_t)511;
  for (int l = 0; l < kCopyLanes; ++l) {
    errs[l] = hipSuccess;
    th[l] = std::thread([&, l]() {
      if (hipSetDevice(c->device) != hipSuccess) {
        errs[l] = hipErrorInvalidDevice;
        return;
      }
      const size_t lo = std::min(count, (size_t)l * per_lane);
      const size_t hi = std::min(count, lo + per_lane);
      char* stage = static_cast<char*>(c->out_stage) + (size_t)l * 2 * kCopyBlock;
      const size_t blk = kCopyBlock / sizeof(double);
      hipStream_t st = c->out_stream[l];
      // block k is in flight while block k - 1 is copied out
      size_t issued = lo, drained = lo;
      int slot = 0;
      auto issue = [&]() {
        const size_t m = std::min(blk, hi - issued);
        const hipError_t e = hipMemcpyAsync(stage + (size_t)slot * kCopyBlock, dev + issued,
                                            m * sizeof(double), hipMemcpyDeviceToHost, st);
        if (e != hipSuccess) errs[l] = e;
        issued += m;
        slot ^= 1;
      };
      if (issued < hi) issue();
      while (drained < hi && errs[l] == hipSuccess) {
        const hipError_t e = hipStreamSynchronize(st);  // the block issued last has landed
        if (e != hipSuccess) {
          errs[l] = e;
          break;
        }
        const int ready = slot ^ 1;
        const size_t m = std::min(blk, hi - drained);
        if (issued < hi) issue();                       // next block on its way ...
        memcpy(out + drained, stage + (size_t)ready * kCopyBlock, m * sizeof(double));  // ... during this
        drained += m;
      }
    });
  }
  for (int l = 0; l < kCopyLanes; ++l) th[l].join();
  for (int l = 0; l < kCopyLanes; ++l)
    if (errs[l] != hipSuccess) {
      (void)hipGetLastError();
      return fail(c, PLR_ERR_HIP,
                  std::string("copying results to the host failed: ") + hipGetErrorString(errs[l]));
    }
  return PLR_OK;
}

// The other direction: pageable host memory into the device through the same pinned lanes.
// A job is at most one staging block; `fill` writes job j's bytes into the pinned block it
// is handed (false stops every lane -- the caller has recorded why), the block is sent to
// jobs[j].dev on the lane's stream, and `sent`, when given, queues more work behind that
// transfer on the same stream.  Jobs are dealt to the lanes in turn; a lane's thread fills
// one of its two blocks while the other is in flight.  Job j uses block (j % lanes) * 2 +
// (j / lanes) % 2 of the staging area.
static int lanes_in(plr_ctx* c, const std::vector<InJob>& jobs, const FillFn& fill,
                    const SentFn& sent, const char* what, LaneProgress* prog,
                    const std::function<int()>* conductor) {
  if (jobs.empty()) return PLR_OK;
  if (!c->out_stage) {
    PLR_HIP(c, hipHostMalloc(&c->out_stage, 2 * kCopyLanes * kCopyBlock, hipHostMallocDefault));
    for (int l = 0; l < kCopyLanes; ++l)
      PLR_HIP(c, hipStreamCreateWithFlags(&c->out_stream[l], hipStreamNonBlocking));
  }
  hipError_t errs[kCopyLanes];
  std::atomic<bool> stop(false);
  auto lane = [&](int l) {
    errs[l] = hipSuccess;
    if (hipSetDevice(c->device) != hipSuccess) {
      errs[l] = hipErrorInvalidDevice;
      if (prog) prog->failed.store(true);
      return;
    }
    char* stage = static_cast<char*>(c->out_stage) + (size_t)l * 2 * kCopyBlock;
    hipStream_t st = c->out_stream[l];
    hipEvent_t freed[2] = {nullptr, nullptr};
    if (hipEventCreateWithFlags(&freed[0], hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&freed[1], hipEventDisableTiming) != hipSuccess)
      errs[l] = hipErrorOutOfMemory;
    int slot = 0;
    size_t round = 0;
    for (size_t j = l; j < jobs.size() && errs[l] == hipSuccess && !stop.load();
         j += kCopyLanes, ++round, slot ^= 1) {
      // the block sent from this slot two rounds ago must have left it
      if (round >= 2 && hipEventSynchronize(freed[slot]) != hipSuccess) errs[l] = hipErrorUnknown;
      char* blk = stage + (size_t)slot * kCopyBlock;
      if (!fill(j, blk)) {
        stop.store(true);
        break;
      }
      hipError_t e = hipMemcpyAsync(jobs[j].dev, blk, jobs[j].bytes, hipMemcpyHostToDevice, st);
      if (e == hipSuccess && sent) e = sent(j, st);
      if (e == hipSuccess) e = hipEventRecord(freed[slot], st);
      if (e == hipSuccess && prog) {
        // whoever waits for this job's bytes waits for this event; the count is
        // published only once the record has been issued
        e = hipEventRecord(prog->done[j], st);
        if (e == hipSuccess) prog->issued[l].store(round + 1, std::memory_order_release);
      }
      if (e != hipSuccess) errs[l] = e;
    }
    if (prog && (errs[l] != hipSuccess || stop.load())) prog->failed.store(true);
    if (hipStreamSynchronize(st) != hipSuccess && errs[l] == hipSuccess) errs[l] = hipErrorUnknown;
    for (int k = 0; k < 2; ++k)
      if (freed[k]) (void)hipEventDestroy(freed[k]);
  };
  const int nl = (int)std::min<size_t>(kCopyLanes, jobs.size());
  for (int l = nl; l < kCopyLanes; ++l) errs[l] = hipSuccess;
  std::thread th[kCopyLanes];
  // with a conductor every lane has a thread of its own and the caller's thread
  // conducts (queues the work that follows the transfers, as they are issued)
  const int first_thread = conductor ? 0 : 1;
  for (int l = first_thread; l < nl; ++l) th[l] = std::thread(lane, l);
  int conducted = PLR_OK;
  if (conductor) conducted = (*conductor)();
  else lane(0);
  for (int l = first_thread; l < nl; ++l) th[l].join();
  if (conducted != PLR_OK) return conducted;
  for (int l = 0; l < kCopyLanes; ++l)
    if (errs[l] != hipSuccess) {
      (void)hipGetLastError();
      return fail(c, PLR_ERR_HIP, std::string(what) + ": " + hipGetErrorString(errs[l]));
    }
  return PLR_OK;
}

// Bytes as they lie (the sample text, the labels, a shard at the device's own pitch).
static int copy_bytes_in(plr_ctx* c, const std::vector<CopyPiece>& pieces) {
  size_t total = 0;
  std::vector<InJob> jobs;
  std::vector<const char*> src;
  for (const CopyPiece& p : pieces) {
    total += p.bytes;
    for (size_t at = 0; at < p.bytes; at += kCopyBlock) {
      jobs.push_back({static_cast<char*>(p.dev) + at, std::min(kCopyBlock, p.bytes - at)});
      src.push_back(static_cast<const char*>(p.src) + at);
    }
  }
  if (total < 4 * kCopyBlock) {
    for (const CopyPiece& p : pieces)
      if (p.bytes) PLR_HIP(c, hipMemcpy(p.dev, p.src, p.bytes, hipMemcpyHostToDevice));
    return PLR_OK;
  }
  return lanes_in(
      c, jobs,
      [&](size_t j, char* blk) {
        memcpy(blk, src[j], jobs[j].bytes);
        return true;
      },
      SentFn(), "copying to the device failed", nullptr, nullptr);
}

// Rows [row0, row0 + nrows) of the caller's row-major X (leading dimension ldx) into the
// resident shard.  A strided copy command would move one row per transfer (~1 GB/s), so
// the lanes' threads repack the rows at the pitch they have on the device -- without the
// constant first column when that is not stored, pad columns zeroed -- into their pinned
// blocks and send those as linear copies.  Row-tiled shards: a job's rows go, stored
// columns only, into a block of a staging buffer on the device, and tile_rows, queued
// behind the transfer on the lane's stream, brings them into the layout.  Rows wider
// than a staging block are cut by columns.  With first_column_is_one the threads also
// check the caller's statement; the first row that breaks it is named.
static int copy_rows_in(plr_ctx* c, int64_t row0, int64_t nrows, const double* X, int64_t ldx) {
  const bool tiled = c->lane != nullptr;
  const int skip = c->bias ? 1 : 0;                 // the constant first column stays on the host
  const int64_t sp = tiled ? c->dcols : c->pitch;   // pitch of the rows as they are sent
  const int64_t blk_cols = (int64_t)(kCopyBlock / sizeof(double));
  if (!tiled && !c->bias && ldx == sp && c->dcols == sp)  // as they lie: one linear stretch
    return copy_bytes_in(c, {{c->dX + row0 * sp, X, (size_t)nrows * sp * sizeof(double)}});
  if (tiled && !c->up_dev) {
    if (hipMalloc(&c->up_dev, 2 * kCopyLanes * kCopyBlock) != hipSuccess) {
      (void)hipGetLastError();
      c->up_dev = nullptr;
      return fail(c, PLR_ERR_NOMEM, "cannot allocate the device upload staging buffer");
    }
  }
  struct RowJob {
    int64_t r0, m;   // rows [r0, r0 + m) of this upload ...
    int64_t c0, w;   // ... columns [c0, c0 + w) of the sent row (whole rows unless m == 1)
  };
  std::vector<RowJob> rj;
  std::vector<InJob> jobs;
  if (sp <= blk_cols) {
    const int64_t per = blk_cols / sp;
    for (int64_t r0 = 0; r0 < nrows; r0 += per) rj.push_back({r0, std::min(per, nrows - r0), 0, sp});
  } else {
    for (int64_t r = 0; r < nrows; ++r)
      for (int64_t c0 = 0; c0 < sp; c0 += blk_cols) rj.push_back({r, 1, c0, std::min(blk_cols, sp - c0)});
  }
  jobs.reserve(rj.size());
  for (size_t j = 0; j < rj.size(); ++j) {
    double* dev = tiled ? c->up_dev + ((j % kCopyLanes) * 2 + (j / kCopyLanes) % 2) * (size_t)blk_cols
                        : c->dX + (row0 + rj[j].r0) * c->pitch + rj[j].c0;
    jobs.push_back({dev, (size_t)(rj[j].m * rj[j].w) * sizeof(double)});
  }
  std::atomic<int64_t> bad_row(INT64_MAX);
  const int64_t dcols = c->dcols;
  const bool dense = (skip == 0 && ldx == sp && dcols == sp);  // tiled rows that are already packed
  auto fill = [&](size_t j, char* blk) {
    const RowJob& q = rj[j];
    double* dst = reinterpret_cast<double*>(blk);
    if (dense) {
      memcpy(dst, X + q.r0 * ldx, (size_t)(q.m * sp) * sizeof(double));
      return true;
    }
    for (int64_t r = 0; r < q.m; ++r, dst += q.w) {
      const double* row = X + (q.r0 + r) * ldx;
      if (skip && q.c0 == 0 && row[0] != 1.) {
        int64_t seen = bad_row.load();
        while (q.r0 + r < seen && !bad_row.compare_exchange_weak(seen, q.r0 + r)) {
        }
        return false;
      }
      const int64_t have = std::max<int64_t>(0, std::min(q.w, dcols - q.c0));  // the rest is padding
      if (have) memcpy(dst, row + skip + q.c0, (size_t)have * sizeof(double));
      for (int64_t k = have; k < q.w; ++k) dst[k] = 0.;
    }
    return true;
  };
  SentFn sent;
  if (tiled) {
    const int np = c->lane->np;
    sent = [&, np](size_t j, hipStream_t st) {
      const int64_t threads = ceil_div(rj[j].m, plr::kWave) * plr::kWave * np;
      hipLaunchKernelGGL(plr::tile_rows, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, st,
                         (const double*)jobs[j].dev, sp, rj[j].m, (int)dcols, c->dX,
                         row0 + rj[j].r0, np);
      return hipGetLastError();
    };
  }
  const int rc = lanes_in(c, jobs, fill, sent, "upload: host-to-device copy failed", nullptr,
                          nullptr);
  if (bad_row.load() != INT64_MAX) {
    // lanes run ahead of each other: an earlier row may break the statement too
    int64_t first = bad_row.load();
    for (int64_t r = 0; r < first; ++r)
      if (X[r * ldx] != 1.) {
        first = r;
        break;
      }
    char b[160];
    snprintf(b, sizeof b, "first_column_is_one is set, but row %lld starts with %.17g",
             (long long)(row0 + first), X[first * ldx]);
    return fail(c, PLR_ERR_INVALID, b);
  }
  return rc;
}

static int predict_rows(plr_ctx* c, PassKind kind, const double* theta, double* out) {
  if (!c) return PLR_ERR_INVALID;
  if (!out && c->n > 0) return fail(c, PLR_ERR_INVALID, "output must not be NULL");
  int rc = run_pass(c, kind, theta, plr::kLossNone, 0., 0.);
  if (rc != PLR_OK) return rc;
  if (c->n > 0 && c->h_pred) {
    copy_host_parallel(out, c->h_pred, (size_t)c->n);
    return PLR_OK;
  }
  if (c->n > 0) return copy_rows_out(c, out, c->d_h, (size_t)c->n);
  return PLR_OK;
}

int plr_predict(plr_ctx* c, const double* theta, double* h_out) {
  return predict_rows(c, kPassPredict, theta, h_out);
}

int plr_predict_linear(plr_ctx* c, const double* theta, double* z_out) {
  return predict_rows(c, kPassPredictLinear, theta, z_out);
}

int plr_probe_read_bandwidth(plr_ctx* c, int reps, double* gb_per_s) {
  if (!c) return PLR_ERR_INVALID;
  if (!gb_per_s || reps < 1) return fail(c, PLR_ERR_INVALID, "need reps >= 1 and an output");
  if (!c->have_data || c->n == 0) return fail(c, PLR_ERR_NODATA, "no shard resident");
  PLR_HIP(c, hipSetDevice(c->device));
  const size_t bytes = (size_t)c->n * c->pitch * sizeof(double);
  const int64_t ntiles = (int64_t)(bytes / 8192);
  if (ntiles < 1) return fail(c, PLR_ERR_INVALID, "shard smaller than one 8 KiB tile");
  const int grid = c->num_cu;
  for (int i = 0; i < 2; ++i)
    hipLaunchKernelGGL(plr::read_probe, dim3(grid), dim3(256), 0, c->stream,
                       reinterpret_cast<const plr::v2d*>(c->dX), ntiles, c->d_part_loss);
  PLR_HIP(c, hipEventRecord(c->ev0, c->stream));
  for (int i = 0; i < reps; ++i)
    hipLaunchKernelGGL(plr::read_probe, dim3(grid), dim3(256), 0, c->stream,
                       reinterpret_cast<const plr::v2d*>(c->dX), ntiles, c->d_part_loss);
  PLR_HIP(c, hipGetLastError());
  PLR_HIP(c, hipEventRecord(c->ev1, c->stream));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  float ms = 0.f;
  PLR_HIP(c, hipEventElapsedTime(&ms, c->ev0, c->ev1));
  *gb_per_s = (double)ntiles * 8192.0 * reps / (ms * 1e-3) / 1e9;
  return PLR_OK;
}

int plr_probe_copy_bandwidth(plr_ctx* c, int64_t bytes, int reps, double* gb_per_s) {
  if (!c) return PLR_ERR_INVALID;
  if (!gb_per_s || reps < 1 || bytes < 1)
    return fail(c, PLR_ERR_INVALID, "need bytes >= 1, reps >= 1 and an output");
  PLR_HIP(c, hipSetDevice(c->device));
  void *src = nullptr, *dst = nullptr;
  hipError_t e = hipMalloc(&src, (size_t)bytes);
  if (e == hipSuccess) e = hipMalloc(&dst, (size_t)bytes);
  if (e == hipSuccess) e = hipMemsetAsync(src, 1, (size_t)bytes, c->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, c->stream);
  if (e == hipSuccess) e = hipEventRecord(c->ev0, c->stream);
  for (int i = 0; i < reps && e == hipSuccess; ++i)
    e = hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, c->stream);
  if (e == hipSuccess) e = hipEventRecord(c->ev1, c->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, c->ev0, c->ev1);
  if (src) (void)hipFree(src);
  if (dst) (void)hipFree(dst);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(c, e == hipErrorOutOfMemory ? PLR_ERR_NOMEM : PLR_ERR_HIP,
                std::string("copy probe failed: ") + hipGetErrorString(e));
  }
  *gb_per_s = 2.0 * (double)bytes * reps / (ms * 1e-3) / 1e9;
  return PLR_OK;
}

int plr_synchronize(plr_ctx* c) {
  if (!c) return PLR_ERR_INVALID;
  PLR_HIP(c, hipSetDevice(c->device));
  PLR_HIP(c, hipStreamSynchronize(c->stream));
  PLR_HIP(c, hipDeviceSynchronize());
  return PLR_OK;
}

int plr_get_shape(const plr_ctx* c, int64_t* n, int64_t* d) {
  if (!c) return PLR_ERR_INVALID;
  if (n) *n = c->n;
  if (d) *d = c->d;
  return PLR_OK;
}

int plr_get_timing(const plr_ctx* c, double* last_ms, double* sum_ms, int64_t* launches) {
  if (!c) return PLR_ERR_INVALID;
  if (last_ms) *last_ms = c->last_ms;
  if (sum_ms) *sum_ms = c->sum_ms;
  if (launches) *launches = c->launches;
  return PLR_OK;
}

int plr_set_option(plr_ctx* c, const char* key, int64_t value) {
  if (!c) return PLR_ERR_INVALID;
  if (!key) return fail(c, PLR_ERR_INVALID, "key must not be NULL");
  if (strcmp(key, "team_spin_limit") == 0) {
    if (value < 0 || value > 0xffffffffLL) return fail(c, PLR_ERR_INVALID, "spin limit out of range");
    c->team_spin_limit = (unsigned)value;
    return PLR_OK;
  }
  if (strcmp(key, "team_lag") == 0) {
    if (value < 0 || value > 2) return fail(c, PLR_ERR_INVALID, "team_lag is 0 (by shape), 1 or 2");
    c->opt_team_lag = (int)value;  // takes effect at the next plr_set_data / plr_alloc_data
    return PLR_OK;
  }
  if (strcmp(key, "team_fallback") == 0) {
    c->opt_team_fallback = value != 0;
    return PLR_OK;
  }
  if (strcmp(key, "first_column_is_one") == 0) {
    c->opt_first_col_one = value != 0;  // takes effect at the next plr_set_data / plr_alloc_data
    return PLR_OK;
  }
  if (strcmp(key, "poll_results") == 0) {
    c->opt_poll_results = value != 0;
    return PLR_OK;
  }
  if (strcmp(key, "csv_overlap") == 0) {
    c->opt_csv_overlap = value != 0;
    return PLR_OK;
  }
  if (strcmp(key, "column_blocks_two_sweeps") == 0) {
    c->opt_two_sweeps = value != 0;  // takes effect at the next plr_set_data / plr_alloc_data
    return PLR_OK;
  }
  return fail(c, PLR_ERR_INVALID, std::string("unknown option ") + key);
}

int plr_set_timing(plr_ctx* c, int enabled) {
  if (!c) return PLR_ERR_INVALID;
  c->timing = enabled != 0;
  return PLR_OK;
}

int plr_reset_timing(plr_ctx* c) {
  if (!c) return PLR_ERR_INVALID;
  c->last_ms = c->sum_ms = 0.;
  c->launches = 0;
  return PLR_OK;
}

int plr_loss_grad_noalloc(int device_id, void* hip_stream, const double* dX, const double* dy,
                          int64_t n, int64_t d, int64_t ldx, const double* dtheta,
                          double* dout, unsigned flags) {
  auto bad = [](int code, const std::string& msg) {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    g_create_error = "plr_loss_grad_noalloc: " + msg;
    return code;
  };
  if (device_id < 0 || device_id >= kNaMaxDevices) return bad(PLR_ERR_INVALID, "device_id out of range");
  if (n < 0 || d < 1) return bad(PLR_ERR_INVALID, "need n >= 0 and d >= 1");
  if (ldx < plr::kChunkCols || ldx % plr::kChunkCols != 0 || ldx < d)
    return bad(PLR_ERR_INVALID, "ldx must be a multiple of 128 and >= d");
  if (ldx > kNaMaxPitch) {
    char b[160];
    snprintf(b, sizeof b, "ldx = %lld exceeds the static scratch's limit of %lld columns",
             (long long)ldx, (long long)kNaMaxPitch);
    return bad(PLR_ERR_INVALID, b);
  }
  if (n > (int64_t)((SIZE_MAX / sizeof(double)) / (size_t)ldx))
    return bad(PLR_ERR_INVALID, "n * ldx overflows");
  if ((n > 0 && (!dX || !dy)) || !dtheta || !dout)
    return bad(PLR_ERR_INVALID, "device pointers must not be NULL");
  // the pass loads X 16 bytes per lane; the other operands are read and written as doubles
  if ((reinterpret_cast<uintptr_t>(dX) & 15u) != 0)
    return bad(PLR_ERR_INVALID, "dX must be 16-byte aligned");
  if (((reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(dtheta) |
        reinterpret_cast<uintptr_t>(dout)) & 7u) != 0)
    return bad(PLR_ERR_INVALID, "dy, dtheta and dout must be 8-byte aligned");
  if (flags > plr::kLossSquared) return bad(PLR_ERR_INVALID, "unknown loss flag");
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

  // the caller's current device is left as it was found
  struct DeviceScope {
    int prev = -1;
    ~DeviceScope() {
      if (prev >= 0) (void)hipSetDevice(prev);
    }
  } scope;
  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) {
    (void)hipGetLastError();
    cur = -1;
  }

#define PLR_NA_HIP(call)                                                        \
  do {                                                                          \
    hipError_t e_ = (call);                                                     \
    if (e_ != hipSuccess) {                                                     \
      (void)hipGetLastError();                                                  \
      return bad(PLR_ERR_HIP, std::string(#call " failed: ") + hipGetErrorString(e_)); \
    }                                                                           \
  } while (0)

  if (cur != device_id) {
    PLR_NA_HIP(hipSetDevice(device_id));
    scope.prev = cur;  // -1: there was none to go back to
  }

  // the row pitch is a whole number of chunks, so the variant is the exact
  // one-wave one for ldx / 128 chunks and no lane reads past a row end
  plr_plan::Plan pl;
  if (!plr_plan::plan_width(ldx, pl, n) || pl.path != plr_plan::kPathFused || pl.pitch != ldx ||
      !pl.allch || pl.tail_cols != 0 || pl.theta_len > kNaMaxPitch)
    return bad(PLR_ERR_UNSUPPORTED, "no kernel variant covers this pitch");
  const Shape* v = &kShapes[pl.variant];
  const bool grad = true;
  const pass_fn fn = kFns[pl.variant].fn[grad ? 1 : 0][1];
  if (!fn || v->wcol != 1) return bad(PLR_ERR_UNSUPPORTED, "kernel variant lacks this instance");
  const int threads = plr::kWave * v->wcol * v->wrow;

  unsigned char* base = nullptr;
  int num_cu = 0, occ = 0;
  {
    // First call on this device (and first call with this pitch on it): the
    // device's own address of the static array, its compute-unit count and the
    // variant's occupancy are looked up once and kept.  These look-ups are not
    // stream work; a caller that captures the stream makes one call per pitch
    // it will use before the capture begins.
    std::lock_guard<std::mutex> lock(g_na_mutex);
    if (!g_na_ptr[device_id]) {
      hipDeviceProp_t prop;
      PLR_NA_HIP(hipGetDeviceProperties(&prop, device_id));
      if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return bad(PLR_ERR_UNSUPPORTED, std::string("device is ") + prop.gcnArchName +
                                            "; this library carries gfx950 code only");
      unsigned char* ptr = nullptr;
      PLR_NA_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
      if (!ptr) return bad(PLR_ERR_HIP, "hipGetSymbolAddress returned a null address");
      g_na_num_cu[device_id] = prop.multiProcessorCount;
      g_na_ptr[device_id] = ptr;
    }
    // (a pitch may map to two variants, by shard size: the slot remembers
    // which one its figure belongs to)
    int& slot = g_na_occ[device_id][ldx / plr::kChunkCols];
    const int tag = (pl.variant + 1) << 8;
    if ((slot & ~0xff) != tag) {
      int o = 0;
      PLR_NA_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &o, reinterpret_cast<const void*>(fn), threads, 0));
      if (o < 1) return bad(PLR_ERR_HIP, "kernel variant does not fit on a compute unit");
      slot = tag | (o > 255 ? 255 : o);
    }
    occ = slot & 0xff;
    base = g_na_ptr[device_id];
    num_cu = g_na_num_cu[device_id];
  }
  double* s_theta = reinterpret_cast<double*>(base + kNaThetaOff);
  double* s_loss = reinterpret_cast<double*>(base + kNaLossOff);
  double* s_part = reinterpret_cast<double*>(base + kNaPartOff);

  const int64_t want = ceil_div(ceil_div(n, v->R), v->wrow);
  int64_t g = std::min<int64_t>((int64_t)num_cu * occ, kNaMaxGrid);
  if (g > want) g = want;
  if (g < 1) g = 1;
  const int grid = (int)g;

  hipLaunchKernelGGL(plr::stage_theta_padded, dim3(2), dim3(256), 0, stream, dtheta, s_theta, d,
                     pl.theta_len);
  PLR_NA_HIP(hipGetLastError());
  if (n > 0) {
    PassArgs pa;
    pa.X = dX;
    pa.y = dy;
    pa.theta = s_theta;
    pa.part_g = s_part;
    pa.part_loss = s_loss;
    pa.h_out = nullptr;
    pa.n = n;
    pa.pitch = ldx;
    pa.width = ldx;
    pa.ntiles = ceil_div(n, v->R);
    pa.nch_rt = pl.nch_rt;
    pa.tail_cols = 0;
    pa.loss_mode = flags;
    pa.identity_link = flags == plr::kLossSquared ? 1 : 0;
    pa.z_buf = nullptr;
    pa.z_accumulate = 0;
    pa.res_in = nullptr;
    pa.theta_bias = nullptr;
    pa.part_res = nullptr;
    hipLaunchKernelGGL(fn, dim3(grid), dim3(threads), 0, stream, pa);
    PLR_NA_HIP(hipGetLastError());
  } else {
    // empty shard: the one partial the finishing kernel reads starts at zero
    hipLaunchKernelGGL(plr::fill_zero, dim3(8), dim3(256), 0, stream, s_part, ldx);
    PLR_NA_HIP(hipGetLastError());
    hipLaunchKernelGGL(plr::fill_zero, dim3(1), dim3(256), 0, stream, s_loss, (int64_t)1);
    PLR_NA_HIP(hipGetLastError());
  }
  FinishArgs fa;
  fa.part_g = s_part;
  fa.part_loss = s_loss;
  fa.theta = s_theta;
  fa.out = dout;
  fa.pitch = ldx;
  fa.d = d;
  fa.n = n;
  fa.nparts = grid;
  fa.nparts_loss = grid;
  fa.delta_mode = 0;
  fa.have_grad = 1;
  fa.alpha = 0.;
  fa.coff2 = 0.;
  fa.theta_rw = nullptr;
  fa.loss_slot = nullptr;
  fa.part_res = nullptr;
  fa.theta_bias = nullptr;
  fa.done = nullptr;
  fa.seq = 0;
  fa.status_in = nullptr;
  fa.status_out = nullptr;
  hipLaunchKernelGGL(plr::finish_pass, dim3((int)ceil_div(d, plr::kFinCols)),
                     dim3(plr::kFinCols * plr::kFinSlices), 0, stream, fa);
  PLR_NA_HIP(hipGetLastError());
#undef PLR_NA_HIP
  return PLR_OK;
}

const char* plr_kernel_info(const plr_ctx* c) { return c ? c->info.c_str() : ""; }

const char* plr_last_error(const plr_ctx* c) {
  return c ? c->err.c_str() : g_create_error.c_str();
}

const char* plr_version(void) { return "plr 0.1 (gfx950)"; }

}  // extern "C"

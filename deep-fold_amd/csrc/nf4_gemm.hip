// Chunked-prefill NF4 GEMM for gfx950: y[M,N] = dequant(W[M,K]) @ x[K,N],
// N <= 32 token columns, on the CDNA4 bf16 matrix cores.  Also the launch
// planner, the split-K reduction and the chr_nf4_gemm* entry points.
// Replaces gpu/nf4/nf4_gemm.cu:665-678 (reduce), 933-1450 (prefill tiles),
// 1497-1785 (tuning, planner, entry points).
//
// Two tile kernels share the planner, the row blocks (128 rows), the split-K partials and the
// reduces.  gemm_rows (described where it is defined) serves every launch whose K slice is at
// most four K tiles long, which is what the planner's split-K produces; gemm_mfma, described
// here, serves the longer slices of launches without a workspace.
//
// Tile.  A workgroup is four wavefronts and owns 128 output rows; each
// wavefront owns 32 of them and all N columns, accumulating one 32x32 fp32
// tile with v_mfma_f32_32x32x16_bf16.  For that instruction lane l supplies
// A[row l%32][k 8*(l/32) .. +8) and B[k 8*(l/32) .. +8)][col l%32], eight
// consecutive k each, i.e. exactly one packed dword of codes on the A side.
//
// Weights.  The MFMA layout wants 32 different rows per instruction, which read
// straight from global memory would be a 64-line gather.  Instead a wavefront
// fetches its 32 rows x 128 bytes of a K tile with four fully coalesced loads
// (eight rows of one 128-byte line each), one tile ahead of the arithmetic, and
// passes them through a private LDS area (row stride 144 bytes, conflict-free for
// the 16-byte reads); the group scales of the tile travel the same way.  A lane
// then takes 16 bytes (32 codes) of its row per 64-wide K step, rebuilds
// bf16(LUT*scale) in registers (one byte-select AND and one LDS lookup per code,
// the 16 levels at LDS address 0) and feeds four MFMAs.
//
// Activations.  The tile [BK=256, N] is contiguous in x; every thread fetches its
// 16-byte vectors of the next tile while the current one is multiplied, then
// scatters them into LDS transposed to [32][BK+8] bf16 (token-major, padded so the
// 16-byte B reads of 32 lanes fall in distinct banks).  Columns >= N and rows >= K
// are zero, so padding codes and unused MFMA columns contribute nothing.
//
// Split-K over grid.y writes fp32 partials [split][M][N] to the caller's
// workspace; a second kernel adds them in split order (deterministic) and
// rounds once to bf16.
//
// Numerics (gpu/nf4/nf4_gemm.cu:168-172, 312-323): weight = bf16(LUT*scale),
// bf16 x bf16 products, fp32 accumulate, one bf16 rounding of y.

#include "nf4_common.h"

#include <type_traits>

#include <atomic>
#include <mutex>

#include <algorithm>
#include <cstdlib>
#include <utility>

namespace chr {

int gemv_entry(const chr_nf4_dev_t *w, const void *x, void *y, void *stream, const void *add,
               const void *rms_w, float rms_eps, const float *sq_in, float *sq_out);
int gemv_rows_per_wg(int M, int K, int K_pad);
int gemv_threads_per_wg(int M, int K, int K_pad);
int gemv_grid_x(int M, int K, int K_pad);
int gemv_step_codes(int M, int K, int K_pad);
int gemv_lds_bytes(int M, int K, int K_pad);

namespace {

constexpr int kLiveMaxN = 32;
constexpr int kPlanMaxN = 64;

constexpr int kBM = 128;      // rows per workgroup
constexpr int kBK = 256;      // K per staged activation tile
constexpr int kBN = 32;       // token columns of the MFMA tile
// Wavefront groups of a workgroup that take alternate K tiles and add their results
// through LDS.  Two groups were measured slower than one at the 14B shapes (72 KB of LDS
// leaves two workgroups per compute unit and the grid no longer fits one round).
constexpr int kKHalves = 1;
constexpr int kGroupThreads = 256;                    // four wavefronts x 32 rows
constexpr int kGemmBlock = kKHalves * kGroupThreads;
constexpr int kXPad = 8;      // bf16 elements of row padding in LDS
constexpr int kXStride = kBK + kXPad;
constexpr int kWRow = kBK / 2 + 16;             // bytes of one staged weight row (padded)
constexpr int kWStage = 32 * kWRow;             // bytes of a wavefront's weight area
constexpr int kGroupsPerTile = kBK / 64;
// codebook + activation tile (NB blocks of 32 columns) + per-wavefront weight and scale
// areas (= sizeof(GemmLds<NB>))
constexpr int kGemmWaves = kGemmBlock / 64;
constexpr int gemm_lds_bytes(int nb) {
  return 64 + kKHalves * nb * kBN * kXStride * 2 + kGemmWaves * kWStage +
         kGemmWaves * 32 * kGroupsPerTile * 2;
}

// The row-streaming tile (gemm_rows): eight wavefronts x 16 rows, one K slice of up to
// four K tiles per workgroup.
constexpr int kRowsWaves = 8;
constexpr int kRowsBlock = kRowsWaves * 64;
constexpr int kRowsStepK = 128;  // k per wavefront step: 16 rows x 64 bytes
constexpr int kRowsMaxTiles = 4;
static_assert(kRowsWaves * 16 == kBM, "both tiles number their row blocks the same way");
// bf16 elements of one token's row of the transposed slice: 4 dwords more than a multiple
// of 64, so the sixteen 16-byte B reads of a quarter wavefront fall in 64 different banks
constexpr int rows_x_stride(int tps) { return tps * kBK + kXPad; }
// the sixteen levels at LDS address 0 (lookup8_lds0), then nc blocks of sixteen token rows
constexpr int rows_lds_bytes(int nc, int tps) { return 64 + nc * 16 * rows_x_stride(tps) * 2; }
// pairs of 16-byte activation vectors a thread stages (N = 16 nc at most)
constexpr int rows_x_items(int nc, int tps) {
  return (tps * (kBK / 2) * 2 * nc + kRowsBlock - 1) / kRowsBlock;
}
// 64 token rows of four tiles would not leave room for two workgroups per compute unit
constexpr int rows_max_tiles(int nc) { return nc == 4 ? 2 : kRowsMaxTiles; }
constexpr int rows_col_blocks(int N) { return N <= 16 ? 1 : (N <= 32 ? 2 : 4); }

// The stream tile (gemm_stream below): sixteen wavefronts, eight staging and eight multiplying,
// on 32 or 64 rows and all of K; the pair table, two chunks of x and of weights and the rows'
// scales in LDS; three or four chunks of loads in registers.
constexpr int kStreamBlock = 1024;
constexpr int kStreamStagers = 512;  // threads of the wavefronts that stage (the other eight multiply)
constexpr int kStreamRows = 32;
constexpr int kStreamChunkK = 512;
// Chunks of loads a staging thread keeps in flight in registers.  Two: with four (three at 32
// and 64 columns) a compute unit had 64 to 100 KB on the way, and this memory system serves a
// launch fastest with about 32 KB per compute unit in flight (the GEMV's ring: 2 KB a
// wavefront).  Measured at 4 (3) / 2 / 1, us per launch: 7168x5120 N = 8 10.1 / 9.6 / 12.5, N = 16
// 10.7 / 10.0 / 11.9, N = 32 12.7 / 11.9 / 13.5, N = 64 20.5 / 19.8 / 20.2; 13824x5120 15.8 / 14.6 /
// 15.5, 16.5 / 15.3 / 15.4, 17.4 / 16.4 / 16.8, 22.7 / 22.5 / 25.0; 5120x13824 17.2 / 16.2 / 16.6,
// 18.1 / 17.0 / 17.2, 19.4 / 18.4 / 18.7, 27.4 / 27.3 / 29.0.
constexpr int kStreamRing = 2;
constexpr int kStreamBodies = 12;   // chunks of the longest K the tile takes, written out one by one
constexpr int kStreamMaxGroups = kStreamBodies * kStreamChunkK / 64;  // groups of the longest K
constexpr int kStreamXS = kStreamChunkK + kXPad;       // bf16 elements of a token row of one chunk
constexpr int kStreamXBytes = 32 * kStreamXS * 2;      // one chunk of x, 32 token rows
constexpr int kStreamWStride = kStreamChunkK / 2 + 16; // bytes of a staged weight row
constexpr int kStreamTableBytes = 256 * 32 * 4;  // the pair table, 32 copies (see fill_pair_table32)
constexpr int kStreamWBytes = kStreamRows * kStreamWStride;  // a chunk of weights of 32 rows
// rb: 32-row blocks of a workgroup (1 or 2)
constexpr int stream_scale_bytes(int rb) { return kStreamMaxGroups * kStreamRows * rb * 2; }
constexpr int stream_lds_bytes(int rb) {
  return kStreamTableBytes + 2 * kStreamXBytes + 2 * rb * kStreamWBytes + stream_scale_bytes(rb);
}
static_assert(stream_lds_bytes(2) <= 160 * 1024, "LDS of a compute unit");
// The same tile at exactly 64 columns (gemm_stream64 below): 64 rows, chunks of 256.
constexpr int kWideChunkK = 256;
constexpr int kWideBodies = 20;  // chunks of the longest K (of one split) the tile takes
constexpr int kWideRows = 64;
constexpr int kWideXS = kWideChunkK + kXPad;           // bf16 elements of a token row of one chunk
constexpr int kWideXBytes = 64 * kWideXS * 2;          // one chunk of x, 64 token rows
constexpr int kWideWStride = kWideChunkK / 2 + 16;     // bytes of a staged weight row
constexpr int kWideWBytes = kWideRows * kWideWStride;  // a chunk of weights
constexpr int kWideMaxGroups = kWideBodies * kWideChunkK / 64;
constexpr int kWideScaleBytes = kWideMaxGroups * kWideRows * 2;
constexpr int kWideLdsBytes = kStreamTableBytes + 2 * kWideXBytes + 2 * kWideWBytes + kWideScaleBytes;
static_assert(kWideLdsBytes <= 160 * 1024, "LDS of a compute unit");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct Tuning {
  int path;
  int split_k;
  int one_wave;
};

int env_int(const char *name, int dflt) {
  const char *e = std::getenv(name);
  if (e == nullptr || e[0] == '\0') {
    return dflt;
  }
  return std::atoi(e);
}

// Which tile a launch runs: the row-streaming one whenever its K slice is short enough to be
// requested whole.  CHR_NF4_GEMM_ROWS=0 keeps every launch on the K-tiled kernel.
bool rows_kernel_serves(int N, int tiles_per_split) {
  static const bool on = env_int("CHR_NF4_GEMM_ROWS", 1) != 0;
  return on && tiles_per_split <= rows_max_tiles(rows_col_blocks(N));
}

// The stream tile takes chunks of 8..32 columns in whole 16-byte vectors when K_pad is a
// multiple of kBK (the four group scales of a row and K tile are then one aligned 8-byte load;
// gemm_launch checks the pointer), unless a split is forced (it has none), and when K is one
// pass of its written-out chunks (K_pad <= 6144).  Its workgroups hold a compute unit each:
// 32 rows each while the launch then runs in one round, else 64 rows (every x operand feeds
// two weight operands) up to two rounds.  Measured at 14B shapes, N = 8 / 16 / 32, against
// the split tiles with their reduce: q/k/v (7168x5120) 10.9 / 11.9 / 15.7 us against 15.1 /
// 16.0 / 18.5; o (5120x5120) 10.0 / 11.2 / 14.8 against 12.7 / 13.5 / 15.8; gate or up
// (13824x5120, 64 rows) 16.6 / 17.1 / 20.3 against 20.9 / 20.9 / 24.0; gate+up stacked
// (27648 rows, 64 rows, two rounds) 32.8 / 33.6 / 40.2 against 33.6 / 37.0 / 42.6.  Not down
// (K = 13824).  With 64 rows where 32 fill one round q/k/v takes 14.9 / 15.6 / 18.8 (half
// the compute units idle).  CHR_NF4_GEMM_STREAM=0 leaves everything to the two older tiles,
// whose weights are bf16(level * scale) as in the reference's kernel
// (gpu/nf4/nf4_gemm.cu:312-323).
// -1: never, 0: where the cost model below prefers it to the split tiles, 1: wherever it fits.
// Starts from CHR_NF4_GEMM_STREAM (0: never, 2: wherever it fits); chr_nf4_gemm_stream_policy
// changes it.
std::atomic<int> &stream_policy() {
  static std::atomic<int> policy{[] {
    const int e = env_int("CHR_NF4_GEMM_STREAM", 1);
    return e == 0 ? -1 : (e == 2 ? 1 : 0);
  }()};
  return policy;
}

bool stream_columns(int N) {
  return stream_policy().load(std::memory_order_relaxed) >= 0 &&
         ((N >= 8 && N <= 32 && (N & 7) == 0) || N == 64);
}

Tuning &tuning() {
  static Tuning t = [] {
    Tuning init{};
    init.path = env_int("CHR_NF4_PATH", 0);
    init.split_k = env_int("CHR_NF4_SPLIT_K", 0);
    init.one_wave = env_int("CHR_NF4_ONE_WAVE", 0);
    if (init.path < 0 || init.path > 2) init.path = 0;
    if (init.split_k < 0) init.split_k = 0;
    if (init.one_wave < 0) init.one_wave = 0;
    return init;
  }();
  return t;
}


int resolved_one_wave() {
  const int w = tuning().one_wave;
  return w > 0 ? w : device_cu_count();
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// How the stream tile takes a launch: rb = 32-row blocks of a workgroup (0: another tile
// serves the launch), split = workgroups that share a row block's K (grid.y), chunks = 512-wide
// chunks of the longest split.
struct StreamPlan {
  int rb, split, chunks;
};

constexpr int64_t kStreamMinCodes = int64_t{1} << 24;
constexpr int64_t kStreamMinCodes64 = int64_t{1} << 20;  // at 64 columns
constexpr int kArriveSlots = 512;    // owners of a row of arrival counts: streams, and captures in progress
constexpr int kArriveBlocks = 1024;  // row blocks of a launch whose splits meet in the tile

// blocks32, blocks64: 32- and 64-row blocks of the launch (summed over its stacked matrices).
// Picks, among the forms that fit (at most 12 chunks a workgroup; splits only when all
// the caller brought a workspace; at most four rounds of workgroups, and more than one only
// with 3072 of K or more to spread a round's fixed time over and the rounds four fifths full,
// and splits over several rounds only from 24 columns on), the one a cost model fitted to measurements calls cheapest, in hundredths of a
// microsecond: a round of 32-row workgroups 4.5 us + 0.50 / 0.52 / 0.62 / 0.73 us a chunk at
// 8 / 16 / 24 / 32 columns, of 64-row workgroups 6.0 us + 0.86 / 0.93 / 1.00 / 1.06 us a chunk
// (refitted with two chunks of loads in flight per staging thread; before, 5.2 + 0.55 .. 1.06
// and 6.5 + 1.00 .. 1.38),
// 2.3 us for the meeting of a split's partials (at most 8 splits; a split has to win by 3%).
// codes: weights of the launch; with 2^24 or fewer the split tiles keep it (measured at
// 8 / 32 columns, this tile against those: 256x5120 8.2 / 8.8 us against 7.5 / 8.5, 2048x2048
// 6.9 / 9.0 against 7.2 / 8.2, 4096x4096 9.0 / 12.2 against 8.9 / 11.5, 1024x13824 10.6 /
// 18.7 against 10.5 / 12.4; above, 3072x8192 11.0 / 15.2 against 12.1 / 15.1 and the 14B
// shapes below).  At 64 columns, where the split tiles are slower, above 2^20 weights
// (512x2048 14.9 us against 17.7, 2560x2048 13.6 against 19.1, 4096x4096 16.3 against 20.5;
// 256x1024 10.9 against 10.4).  At the 14B shapes:
// q/k/v and o 32 rows x all of K up to 32 columns (o at 32 columns: 11.7 us against 12.4 with
// 64 rows x 3 splits), 64 rows x 2 or 3 splits at 64; gate or up 64 rows; gate+up stacked 64 rows in two
// rounds; down (K = 13824) 64 rows x 3 splits.  CHR_NF4_GEMM_STREAM_ROWS=32 or 64 allows only
// that form, CHR_NF4_GEMM_STREAM_SPLIT=0 no splits.
StreamPlan stream_plan(int N, int K_pad, int blocks32, int blocks64, int have_ws, int64_t codes) {
  static const int only = env_int("CHR_NF4_GEMM_STREAM_ROWS", 0);
  static const bool splits = env_int("CHR_NF4_GEMM_STREAM_SPLIT", 1) != 0;
  StreamPlan best{0, 1, 0};
  if (!stream_columns(N) || tuning().split_k != 0 || K_pad % kBK != 0) {
    return best;
  }
  static constexpr int kFixed[2] = {450, 600};
  static constexpr int kChunk[2][4] = {{50, 52, 62, 73}, {86, 93, 100, 106}};
  constexpr int kWideChunk = 110;  // a 256-wide chunk of the 64-column form
  constexpr int kMeet = 230, kMaxSplit = 8;
  const int cus = resolved_one_wave();
  const bool wide = N == 64;  // 64 rows and chunks of 256 only
  const int n_ch = ceil_div(K_pad, wide ? kWideChunkK : kStreamChunkK);
  const int bodies = wide ? kWideBodies : kStreamBodies;
  int best_cost = 0;
  for (int rb = wide ? 2 : 1; rb <= 2; ++rb) {
    if (only != 0 && only != kStreamRows * rb) {
      continue;
    }
    const int blocks = rb == 1 ? blocks32 : blocks64;
    for (int split = 1; split <= std::min(n_ch, kMaxSplit); ++split) {
      const int chunks = ceil_div(n_ch, split);
      if (ceil_div(n_ch, chunks) != split || chunks > bodies) {
        continue;  // (the same chunks with fewer workgroups comes first; too long a K)
      }
      const int rounds = ceil_div(blocks * split, cus);
      if (rounds > 4 || (split > 1 && (!splits || !have_ws || blocks > kArriveBlocks))) {
        continue;
      }
      // more than one round of workgroups: only long ones (22016x2048 in two rounds of 4
      // chunks: 18.1 / 22.1 us against 14.1 / 20.3) that fill the rounds to four fifths
      if (rounds > 1 && (chunks * (wide ? kWideChunkK : kStreamChunkK) < 6 * kStreamChunkK ||
                         blocks * split * 5 < rounds * cus * 4 || (split > 1 && N < 24))) {
        continue;  // (6144x16384 at 8 columns, 5 splits in two rounds: 28.2 us against 23.8)
      }
      int cost = rounds * (kFixed[rb - 1] + chunks * (wide ? kWideChunk : kChunk[rb - 1][N / 8 - 1]));
      if (split > 1) {
        cost += kMeet;
        cost += cost / 32;
      }
      if (best.rb == 0 || cost < best_cost) {
        best = StreamPlan{rb, split, chunks};
        best_cost = cost;
      }
    }
  }
  if (codes <= (wide ? kStreamMinCodes64 : kStreamMinCodes) && only == 0 &&
      stream_policy().load(std::memory_order_relaxed) == 0) {
    best.rb = 0;
  }
  if (codes >= (int64_t{1} << 33)) {
    best.rb = 0;  // (the tile addresses a matrix's packed bytes with 32-bit offsets)
  }
  return best;
}

// Split-K.  A workgroup is quickest with about three K tiles (measured at every 14B linear
// shape: fewer tiles leave the fetch latency uncovered, more leave compute units idle), so
// split = ceil(n_ktiles / 3) -- but no more splits than it takes to reach a target number of
// workgroups, because every split writes and re-reads M*N fp32 partials: three workgroups per
// compute unit for chunks of up to 32 columns, 1.6 for wider ones (whose partials are twice
// as large; a 27648-row gate+up stack at N=64 takes 65 us with 2 splits, 74 with 4, 87 with
// 10).  split is recomputed from tiles_per_split so the pair always agrees with what the
// kernel indexes (gpu/nf4/nf4_gemm.cu:1526-1543).
constexpr int kTilesPerSplit = 3;
constexpr int kMaxAutoSplit = 32;

// Chunks of up to 32 columns run the row-streaming tile, whose workgroups (one slice of 1..4
// K tiles each) all start at once: what a launch costs is the work of the busiest compute
// unit, ceil(workgroups / compute units) slices, plus what every split adds to the partials
// and their reduce.  Measured per K tile of a slice ~2 us, per split ~0.2 us, and a launch
// that leaves one workgroup per compute unit (nothing to overlap its fetch with) ~1.4 times
// its tiles: 5120x5120 takes 10 splits (15.3 us at N=32) where "three tiles per workgroup"
// gave 7 (280 workgroups on 256 units: 16.9 us); 7168x5120 keeps 7, 5120x13824 keeps 18.
// Ties go to the longer slice (fewer partials).  fallback: the split for slices this tile
// cannot take (more than 4 x 32 K tiles).
int pick_split_rows(int grid_x, int n_ktiles, int cus, int fallback) {
  int best = 0, best_cost = 0;
  for (int tps = 1; tps <= kRowsMaxTiles; ++tps) {
    const int split = ceil_div(n_ktiles, tps);
    if (split > kMaxAutoSplit || ceil_div(n_ktiles, split) != tps) {
      continue;  // too many splits, or the same split as a shorter slice already gave
    }
    const int rounds = ceil_div(grid_x * split, cus);
    const int cost = rounds * tps * (rounds == 1 ? 28 : 20) + split * 2;  // tenths of a us
    if (best == 0 || cost <= best_cost) {
      best = split;
      best_cost = cost;
    }
  }
  return best > 0 ? best : fallback;
}

void pick_split(int grid_x, int n_ktiles, int N, int have_ws, int *split, int *tiles_per_split) {
  const Tuning &t = tuning();
  int want = 1;
  if (have_ws) {
    const int cus = resolved_one_wave();
    const int target = N > kBN ? cus * 8 / 5 : cus * 3;
    const int by_grid = std::max(1, ceil_div(target, grid_x));
    const int by_tiles = ceil_div(n_ktiles, kTilesPerSplit);
    want = t.split_k > 0 ? t.split_k : std::min(kMaxAutoSplit, std::min(by_tiles, by_grid));
    if (t.split_k == 0 && N <= kBN) {
      want = pick_split_rows(grid_x, n_ktiles, cus, want);
    }
  }
  want = std::max(1, std::min(want, n_ktiles));
  const int tps = ceil_div(n_ktiles, want);
  *tiles_per_split = tps;
  *split = ceil_div(n_ktiles, tps);
}

int plan_impl(const chr_nf4_dev_t &h, int32_t N, int32_t have_ws, chr_nf4_plan_t *out) {
  chr_nf4_plan_t p{};
  if (N == 1) {
    // Row-streaming GEMV: every wavefront walks whole rows, no split-K.  bm is the rows a
    // workgroup covers per pass (the staged kernel, one workgroup per compute unit, makes
    // ceil(M / bm / grid_x) passes).
    p.path = 1;
    p.bm = gemv_rows_per_wg(h.M, h.K, h.K_pad);
    p.bk = gemv_step_codes(h.M, h.K, h.K_pad);
    p.block = gemv_threads_per_wg(h.M, h.K, h.K_pad);
    p.grid_x = gemv_grid_x(h.M, h.K, h.K_pad);
    p.grid_y = 1;
    p.n_ktiles = ceil_div(h.K_pad, p.bk);
    p.tiles_per_split = p.n_ktiles;
    p.smem_bytes = gemv_lds_bytes(h.M, h.K, h.K_pad);
    p.ws_floats = 0;
  } else {
    p.path = N <= 16 ? 2 : (N <= 32 ? 3 : 4);
    p.bm = kBM;
    p.bk = kBK;
    p.block = kGemmBlock;
    p.grid_x = ceil_div(h.M, kBM);
    p.n_ktiles = ceil_div(h.K_pad, kBK);
    pick_split(p.grid_x, p.n_ktiles, N, have_ws, &p.grid_y, &p.tiles_per_split);
    p.smem_bytes = gemm_lds_bytes(N <= 32 ? 1 : 2);
    const StreamPlan st =
        stream_plan(N, h.K_pad, ceil_div(h.M, kStreamRows), ceil_div(h.M, 2 * kStreamRows), have_ws,
                    static_cast<int64_t>(h.M) * h.K_pad);
    if (st.rb != 0) {
      p.bm = kStreamRows * st.rb;
      p.block = kStreamBlock;
      p.grid_x = ceil_div(h.M, p.bm);
      p.grid_y = st.split;
      p.tiles_per_split = N == 64 ? st.chunks : std::min(2 * st.chunks, p.n_ktiles);
      p.smem_bytes = N == 64 ? kWideLdsBytes : stream_lds_bytes(st.rb);
    } else if (rows_kernel_serves(N, p.tiles_per_split)) {
      p.block = kRowsBlock;
      p.smem_bytes = rows_lds_bytes(rows_col_blocks(N), p.tiles_per_split);
    }
    if (p.grid_y > 1) {
      p.ws_floats = static_cast<int64_t>(p.grid_y) * h.M * N;
    }
  }
  p.ctas = p.grid_x * p.grid_y;
  *out = p;
  return 0;
}

int check_args(const chr_nf4_dev_t *w, int32_t N, bool need_ptrs, chr_nf4_dev_t *h_out,
               int32_t max_n) {
  if (w == nullptr) {
    return -1;
  }
  if (N < 1 || N > max_n) {
    return -2;
  }
  const chr_nf4_dev_t h = *w;
  if (h.M < 1 || h.K < 1) {
    return -3;
  }
  if (need_ptrs && (h.packed == nullptr || h.scale == nullptr)) {
    return -3;
  }
  if (!k_pad_ok(h.K, h.K_pad)) {
    return -4;
  }
  *h_out = h;
  return 0;
}

// Up to three matrices that share x, K and the chunk (q, k and v of one layer): their row
// blocks are numbered through on grid.x, their outputs stacked in y and in the partials.
struct GemmSegs {
  const uint8_t *packed[3];
  const uint16_t *scale[3];
  int M[3];       // rows of each matrix
  int blocks[3];  // row blocks (of kBM rows) of each
  int row0[3];    // first output row of each
  // the stream tiles: workgroups that share K (grid.y) and the chunks each of them takes, from
  // the host (read from the grid size, a hidden kernel argument, and divided in the kernel they
  // were a trip to the scalar cache and an integer division ahead of the first requests)
  int splits, per_split;
};

template <int NB>
struct GemmLds {
  float lut[16];                                  // at LDS address 0 (lookup8)
  __attribute__((aligned(16))) uint16_t xs[kKHalves][NB * kBN * kXStride];
  __attribute__((aligned(16))) uint8_t w[kGemmWaves][kWStage];
  uint16_t sc[kGemmWaves][32 * kGroupsPerTile];
};
static_assert(sizeof(GemmLds<1>) == gemm_lds_bytes(1) && sizeof(GemmLds<2>) == gemm_lds_bytes(2),
              "the planner reports these sizes");
static_assert(kKHalves == 1, "the two-group reduction was written for one column block");

// Activation vectors of one K tile held by a thread between fetch and scatter.  The tile
// x[k0 .. k0+kBK) x [0, N) is kBK*N contiguous bf16; vector v of a thread holds flat
// elements 8v .. 8v+7, element f being (k0 + f / N, f % N).
template <int NB>
struct XRegs {
  uint32_t d[16 * NB];  // up to 4 NB 16-byte vectors (N = 32 NB), as plain dwords
};

// Vector staging of the activation tile (N in {8, 16, 32, 64}).  An item is a pair of rows
// (k, k+1) and one 8-column vector q: two 16-byte loads, which are interleaved into eight
// dwords {x[k][n], x[k+1][n]} and stored at xs[n][k/2], one 32-bit store each.  Items are dealt
// to lanes so that the 64 stores of a wavefront instruction fall into 64 different LDS banks
// (a column row is 132 dwords = 4 mod 64: bank = 4n + k/2 mod 64).
//   N >= 16: lane -> k pair 32a + (lane & 31), vector 2b + (lane >> 5), a = I % 4, b = I / 4
//   N == 8 : lane -> k pair 64I + lane, vector 0
// with I = wavefront + 4 rep numbering the wavefront instructions of the tile.
__device__ __forceinline__ bool x_item(int N, int I, int lane, int &kp, int &q) {
  if (N == 8) {
    kp = 64 * I + lane;
    q = 0;
    return I < 2;
  }
  kp = 32 * (I & 3) + (lane & 31);
  q = 2 * (I >> 2) + (lane >> 5);
  return I < N / 4;  // 128 k pairs x N/8 vectors = 16 N items = N/4 instructions
}

template <bool VEC, int NB>
__device__ __forceinline__ void fetch_x(XRegs<NB> &r, const uint16_t *__restrict__ x, int k0, int K,
                                        int N, int tid) {
  if constexpr (VEC) {
    const int wave = tid >> 6, lane = tid & 63;
#pragma unroll
    for (int rep = 0; rep < 2 * NB; ++rep) {
      // Every load is issued whatever the item: a load under a branch is waited for where
      // the branch ends, which would put the whole fetch in front of the arithmetic it is
      // meant to overlap.  Items past the tile read vector 0 of a valid row, rows >= K read
      // row K - 1; both are replaced by zeros afterwards.
      int kp, q;
      const bool item = x_item(N, wave + 4 * rep, lane, kp, q);
      const int k = k0 + 2 * kp;
      const int qv = item ? q : 0;
      uint4 a = *reinterpret_cast<const uint4 *>(x + static_cast<size_t>(min(k, K - 1)) * N + 8 * qv);
      uint4 b =
          *reinterpret_cast<const uint4 *>(x + static_cast<size_t>(min(k + 1, K - 1)) * N + 8 * qv);
      // masks, not branches: a conditional assignment compiles to a branch behind the load
      const uint32_t ka = item && k < K ? ~0u : 0u;
      const uint32_t kb = item && k + 1 < K ? ~0u : 0u;
      a = make_uint4(a.x & ka, a.y & ka, a.z & ka, a.w & ka);
      b = make_uint4(b.x & kb, b.y & kb, b.z & kb, b.w & kb);
      r.d[8 * rep + 0] = a.x;
      r.d[8 * rep + 1] = a.y;
      r.d[8 * rep + 2] = a.z;
      r.d[8 * rep + 3] = a.w;
      r.d[8 * rep + 4] = b.x;
      r.d[8 * rep + 5] = b.y;
      r.d[8 * rep + 6] = b.z;
      r.d[8 * rep + 7] = b.w;
    }
  } else {
    (void)r;
  }
}

template <bool VEC, int NB>
__device__ __forceinline__ void scatter_x(const XRegs<NB> &r, const uint16_t *__restrict__ x,
                                          uint16_t *xs, int k0, int K, int N, int tid) {
  if constexpr (VEC) {
    const int wave = tid >> 6, lane = tid & 63;
    uint32_t *xd = reinterpret_cast<uint32_t *>(xs);
#pragma unroll
    for (int rep = 0; rep < 2 * NB; ++rep) {
      int kp, q;
      if (x_item(N, wave + 4 * rep, lane, kp, q)) {
        uint32_t *dst = xd + (8 * q) * (kXStride / 2) + kp;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t a = r.d[8 * rep + e], b = r.d[8 * rep + 4 + e];
          dst[(2 * e) * (kXStride / 2)] = (a & 0xFFFFu) | (b << 16);
          dst[(2 * e + 1) * (kXStride / 2)] = (a >> 16) | (b & 0xFFFF0000u);
        }
      }
    }
  } else {
    // any N, any alignment: element by element
    for (int i = tid; i < kBK * N; i += kGroupThreads) {
      const int kk = i / N;
      const int n = i - kk * N;
      const int k = k0 + kk;
      xs[n * kXStride + kk] = k < K ? x[static_cast<size_t>(k) * N + n] : static_cast<uint16_t>(0);
    }
  }
}

// The 32 rows x 128 bytes of one K tile that a wavefront multiplies, as fetched: load j
// covers rows 8j .. 8j+7, lane l the 16 bytes at offset 16*(l%8) of row 8j + l/8.
struct WRegs {
  uint32_t d[16];
  uint32_t sc;  // two adjacent group scales of row l/2 (groups 2*(l%2), +1 of the tile)
};

__device__ __forceinline__ void fetch_w(WRegs &r, const uint8_t *__restrict__ packed,
                                        const uint16_t *__restrict__ scale, int row_base, int M,
                                        int K_pad, int k0, int lane) {
  const int row_bytes = K_pad >> 1;
  const int col = (k0 >> 1) + ((lane & 7) << 4);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = min(row_base + 8 * j + (lane >> 3), M - 1);
    // unconditional (see fetch_x): past the end of the row its last 16 bytes are read and
    // replaced by the code of 0.0
    uint4 t = *reinterpret_cast<const uint4 *>(packed + static_cast<size_t>(row) * row_bytes +
                                               min(col, row_bytes - 16));
    const uint32_t pad = col >= row_bytes ? ~0u : 0u;  // a mask, not a branch
    const uint32_t fill = 0x77777777u & pad;
    t = make_uint4((t.x & ~pad) | fill, (t.y & ~pad) | fill, (t.z & ~pad) | fill,
                   (t.w & ~pad) | fill);
    r.d[4 * j + 0] = t.x;
    r.d[4 * j + 1] = t.y;
    r.d[4 * j + 2] = t.z;
    r.d[4 * j + 3] = t.w;
  }
  const int srow = min(row_base + (lane >> 1), M - 1);
  const int g = (k0 >> 6) + ((lane & 1) << 1);
  const int groups = K_pad >> 6;
  const uint16_t *sp = scale + static_cast<size_t>(srow) * groups;
  const uint32_t l0 = sp[min(g, groups - 1)], l1 = sp[min(g + 1, groups - 1)];
  const uint32_t s0 = g < groups ? l0 : 0u;
  const uint32_t s1 = g + 1 < groups ? l1 : 0u;
  r.sc = s0 | (s1 << 16);
}

__device__ __forceinline__ void stash_w(const WRegs &r, uint8_t *wst, uint16_t *sst, int lane) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint8_t *dst = wst + (8 * j + (lane >> 3)) * kWRow + ((lane & 7) << 4);
    *reinterpret_cast<uint4 *>(dst) =
        make_uint4(r.d[4 * j + 0], r.d[4 * j + 1], r.d[4 * j + 2], r.d[4 * j + 3]);
  }
  *reinterpret_cast<uint32_t *>(sst + (lane >> 1) * kGroupsPerTile + ((lane & 1) << 1)) = r.sc;
}

// NB: 32-column blocks of the activation tile (1 for N <= 32, 2 for N <= 64); one
// dequantised weight fragment feeds NB MFMAs.
template <bool VEC, int NB>
__global__ __launch_bounds__(kGemmBlock) void gemm_mfma(const GemmSegs segs,
                                                        const uint16_t *__restrict__ x,
                                                        uint16_t *__restrict__ y,
                                                        float *__restrict__ partial, int M_all,
                                                        int K, int K_pad, int N, int n_ktiles,
                                                        int tiles_per_split,
                                                        const uint16_t *__restrict__ bias,
                                                        const uint16_t *res) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  GemmLds<NB> &lds = *reinterpret_cast<GemmLds<NB> *>(lds_raw);
  if (threadIdx.x < 16) {
    lds.lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  // columns >= N of the activation tiles are never written by the scatter: zero them once
  for (int i = threadIdx.x; i < NB * kBN * kXStride / 2; i += kGemmBlock) {
    reinterpret_cast<uint32_t *>(&lds.xs[0][0])[i] = 0u;
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int tid = threadIdx.x;
  // which matrix this row block belongs to, and the block's number inside it
  int bx = static_cast<int>(blockIdx.x);
  int seg = 0;
  if (bx >= segs.blocks[0]) {
    bx -= segs.blocks[0];
    seg = 1;
    if (bx >= segs.blocks[1]) {
      bx -= segs.blocks[1];
      seg = 2;
    }
  }
  const uint8_t *__restrict__ packed = segs.packed[seg];
  const uint16_t *__restrict__ scale = segs.scale[seg];
  const int M = segs.M[seg];
  const int out0 = segs.row0[seg];
  const int row_base = bx * kBM + wave * 32;
  const int khalf = lane >> 5;  // which 32-wide half of a 64-wide K step
  uint8_t *wst = lds.w[wave];
  uint16_t *sst = lds.sc[wave];
  uint16_t *xs = lds.xs[0];

  const int tile0 = blockIdx.y * tiles_per_split;
  const int tile1 = min(tile0 + tiles_per_split, n_ktiles);

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    acc[nb] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  }
  const uint16_t *xl = xs + (lane & 31) * kXStride + khalf * 32;
  const uint8_t *wl = wst + (lane & 31) * kWRow + khalf * 16;
  const uint16_t *sl = sst + (lane & 31) * kGroupsPerTile;

  WRegs wr;
  XRegs<NB> xr;
  if (tile0 < tile1) {
    fetch_w(wr, packed, scale, row_base, M, K_pad, tile0 * kBK, lane);
    fetch_x<VEC, NB>(xr, x, tile0 * kBK, K, N, tid);
  }
  for (int tile = tile0; tile < tile1; ++tile) {
    const int k0 = tile * kBK;
    __syncthreads();  // the previous round's readers are done (and the LUT / zero fill is visible)
    scatter_x<VEC, NB>(xr, x, xs, k0, K, N, tid);
    stash_w(wr, wst, sst, lane);
    __syncthreads();
    {
      // The next tile's trip to memory overlaps this tile's arithmetic.  Unconditional, so
      // that the wait for it lands where the data is used (the last tile fetches itself
      // again and the result is dropped).
      const int kn = min(k0 + kBK, (tile1 - 1) * kBK);
      fetch_w(wr, packed, scale, row_base, M, K_pad, kn, lane);
      fetch_x<VEC, NB>(xr, x, kn, K, N, tid);
    }
    const int kend = min(kBK, K_pad - k0);
    for (int kk = 0; kk < kend; kk += 64) {
      const uint4 pk = *reinterpret_cast<const uint4 *>(wl + (kk >> 1));
      const float s = f16_to_f32(sl[kk >> 6]);
      const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
      // all 32 lookups and the B reads of the step are issued before the first
      // conversion, so their LDS latency is paid once per step
      Levels8 lv[4];
      bf16x8 b[4][NB];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        lv[t] = lookup8_lds0(w[t]);  // lds.lut is at LDS address 0
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          b[t][nb] = *reinterpret_cast<const bf16x8 *>(xl + nb * kBN * kXStride + kk + 8 * t);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        bf16x8 a;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a[j] = static_cast<__bf16>(lv[t].l[j] * s);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[t][nb], acc[nb], 0, 0, 0);
        }
      }
    }
  }

  // acc[nb][i] is C[row 8*(i/4) + 4*(lane/32) + i%4][col 32 nb + lane%32] of the 32-row tile.
  const int rbase = row_base + 4 * (lane >> 5);
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = nb * kBN + (lane & 31);
    if (n < N) {
      if (partial == nullptr) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = rbase + 8 * (i >> 2) + (i & 3);
          if (r < M) {
            // unsplit: the epilogue of reduce_splitk, here (res may alias y: same thread,
            // same element)
            const size_t at = static_cast<size_t>(out0 + r) * N + n;
            uint16_t v = f32_to_bf16(acc[nb][i]);
            if (bias != nullptr) {
              v = f32_to_bf16(bf16_to_f32(v) + bf16_to_f32(bias[out0 + r]));
            }
            if (res != nullptr) {
              v = f32_to_bf16(bf16_to_f32(res[at]) + bf16_to_f32(v));
            }
            y[at] = v;
          }
        }
      } else {
        float *p = partial + static_cast<size_t>(blockIdx.y) * M_all * N;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int r = rbase + 8 * (i >> 2) + (i & 3);
          if (r < M) {
            float *dst = p + static_cast<size_t>(out0 + r) * N + n;
            if constexpr (NB == 2) {
              // wide chunks: full 128-byte runs per row, read once by the reduce
              __builtin_nontemporal_store(acc[nb][i], dst);
            } else {
              *dst = acc[nb][i];
            }
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Row-streaming tile: every weight byte goes from global memory straight into the register
// that feeds the matrix core; only the activations pass through LDS.
//
// A workgroup is eight wavefronts and owns kBM = 128 rows x one K slice of TPS * kBK
// columns (grid.y numbers the slices, so the partials are laid out as for gemm_mfma).  A
// wavefront owns 16 rows and multiplies with v_mfma_f32_16x16x32_bf16, whose A operand is
// 16 rows x 32 k: lane l supplies eight k of row l % 16, the k slots being numbered by
// l / 16.  Which k sits in which slot is free as long as A and B agree, so a step of the
// wavefront is 128 k wide, lane l loads the 16 bytes (32 codes) of row l % 16 at byte
// 16 * (l / 16) of the step -- sixteen rows x 64 contiguous bytes per load instruction --
// and MFMA j of the step takes dword j of every lane: k = 32 * (l / 16) + 8 j .. + 8.  The B
// operand is read from the transposed activation slice at the same k.  All 32 k of a lane
// lie in one 64-wide group, so one scale per lane and step is enough.
//
// Nothing is pipelined: a slice is at most four K tiles, so a lane requests its whole share
// (at most eight 16-byte loads of codes) at the top of the kernel, behind the activation
// requests, and the memory system sees the full grid's weights at once.
//
// Requests past the end of a row or of x are clamped to valid addresses and the activation
// slice holds zeros from k = K on, so they contribute nothing; rows >= M are computed from
// row M - 1 and dropped in the epilogue.

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <bool VEC, int NC, int TPS>
__global__ __launch_bounds__(kRowsBlock) void gemm_rows(const GemmSegs segs,
                                                        const uint16_t *__restrict__ x,
                                                        uint16_t *__restrict__ y,
                                                        float *__restrict__ partial, int M_all,
                                                        int K, int K_pad, int N,
                                                        const uint16_t *__restrict__ bias,
                                                        const uint16_t *res) {
  constexpr int SK = TPS * kBK;
  constexpr int XS = rows_x_stride(TPS);
  constexpr int STEPS = SK / kRowsStepK;
  constexpr int XI = rows_x_items(NC, TPS);
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float *lut = reinterpret_cast<float *>(lds_raw);
  uint16_t *xs = reinterpret_cast<uint16_t *>(lds_raw + 64);
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid < 16) {
    lut[tid] = bits_to_f32(kLutBits[tid]);
  }
  int bx = static_cast<int>(blockIdx.x);
  int seg = 0;
  if (bx >= segs.blocks[0]) {
    bx -= segs.blocks[0];
    seg = 1;
    if (bx >= segs.blocks[1]) {
      bx -= segs.blocks[1];
      seg = 2;
    }
  }
  const uint8_t *__restrict__ packed = segs.packed[seg];
  const uint16_t *__restrict__ scale = segs.scale[seg];
  const int M = segs.M[seg];
  const int out0 = segs.row0[seg];
  const int row_base = bx * kBM + wave * 16;
  const int k0 = static_cast<int>(blockIdx.y) * SK;
  const int r = lane & 15;  // row of the A operand, token of the B operand
  const int g = lane >> 4;  // which quarter of a step's k

  // 1. activation requests: item (k pair kp, vector q) is rows k0 + 2 kp, + 1 of x, columns
  //    8 q .. + 8; q runs fastest over the threads so a row's vectors are fetched together
  const int nv = N >> 3;
  const int n_items = (SK / 2) * nv;
  uint4 xa[XI], xb[XI];
  int xkp[XI], xq[XI];
  if constexpr (VEC) {
#pragma unroll
    for (int it = 0; it < XI; ++it) {
      const int idx = min(tid + it * kRowsBlock, n_items - 1);
      const int kp = idx / nv;
      const int q = idx - kp * nv;
      xkp[it] = kp;
      xq[it] = q;
      const int k = k0 + 2 * kp;
      xa[it] = *reinterpret_cast<const uint4 *>(x + static_cast<size_t>(min(k, K - 1)) * N + 8 * q);
      xb[it] =
          *reinterpret_cast<const uint4 *>(x + static_cast<size_t>(min(k + 1, K - 1)) * N + 8 * q);
    }
  }

  // 2. weight and scale requests, the whole slice of this lane's row
  const int row_bytes = K_pad >> 1;
  const int groups = K_pad >> 6;
  const int row = min(row_base + r, M - 1);
  const uint8_t *prow = packed + static_cast<size_t>(row) * row_bytes;
  const uint16_t *srow = scale + static_cast<size_t>(row) * groups;
  uint4 wq[STEPS];
  uint16_t sc[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int off = min((k0 >> 1) + 64 * s + 16 * g, row_bytes - 16);
    wq[s] = *reinterpret_cast<const uint4 *>(prow + off);
    sc[s] = srow[min((k0 >> 6) + 2 * s + (g >> 1), groups - 1)];
  }

  // 3. token rows N .. 16 NC of the slice are never staged: zero them
  {
    uint32_t *z = reinterpret_cast<uint32_t *>(xs + N * XS);
    const int nz = (16 * NC - N) * (XS / 2);
    for (int i = tid; i < nz; i += kRowsBlock) {
      z[i] = 0u;
    }
  }

  // 4. transpose the activations into LDS: rows k, k + 1 are interleaved into dwords
  //    {x[k][n], x[k + 1][n]} and stored at xs[n][k / 2]
  if constexpr (VEC) {
    uint32_t *xd = reinterpret_cast<uint32_t *>(xs);
#pragma unroll
    for (int it = 0; it < XI; ++it) {
      if (tid + it * kRowsBlock < n_items) {
        const int k = k0 + 2 * xkp[it];
        const bool ka = k < K, kb = k + 1 < K;
        const uint32_t a[4] = {ka ? xa[it].x : 0u, ka ? xa[it].y : 0u, ka ? xa[it].z : 0u,
                               ka ? xa[it].w : 0u};
        const uint32_t b[4] = {kb ? xb[it].x : 0u, kb ? xb[it].y : 0u, kb ? xb[it].z : 0u,
                               kb ? xb[it].w : 0u};
        uint32_t *dst = xd + (8 * xq[it]) * (XS / 2) + xkp[it];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          dst[(2 * e) * (XS / 2)] = (a[e] & 0xFFFFu) | (b[e] << 16);
          dst[(2 * e + 1) * (XS / 2)] = (a[e] >> 16) | (b[e] & 0xFFFF0000u);
        }
      }
    }
  } else {
    // any N, any alignment: element by element
    for (int i = tid; i < SK * N; i += kRowsBlock) {
      const int kk = i / N;
      const int n = i - kk * N;
      const int k = k0 + kk;
      xs[n * XS + kk] = k < K ? x[static_cast<size_t>(k) * N + n] : static_cast<uint16_t>(0);
    }
  }
  __syncthreads();

  // 5. multiply
  f32x4 acc[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const uint16_t *xl = xs + r * XS + 32 * g;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const float sf = f16_to_f32(sc[s]);
    const uint32_t w[4] = {wq[s].x, wq[s].y, wq[s].z, wq[s].w};
#pragma unroll
    for (int jh = 0; jh < 4; jh += 2) {
      // the sixteen lookups and the B reads of two MFMA k blocks are issued before the
      // first conversion, so their LDS latency is paid once per pair
      Levels8 lv[2];
      bf16x8 b[2][NC];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        lv[t] = lookup8_lds0(w[jh + t]);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          b[t][c] = *reinterpret_cast<const bf16x8 *>(xl + c * 16 * XS + kRowsStepK * s +
                                                      8 * (jh + t));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        bf16x8 a;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          a[e] = static_cast<__bf16>(lv[t].l[e] * sf);
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[t][c], acc[c], 0, 0, 0);
        }
      }
    }
  }

  // acc[c][i] is C[row 4 * (lane / 16) + i][col 16 c + lane % 16] of the 16-row tile
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int n = 16 * c + r;
    if (n < N) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int rr = row_base + 4 * g + i;
        if (rr < M) {
          const size_t at = static_cast<size_t>(out0 + rr) * N + n;
          if (partial == nullptr) {
            // unsplit: the epilogue of reduce_splitk, here (res may alias y: same thread,
            // same element)
            uint16_t v = f32_to_bf16(acc[c][i]);
            if (bias != nullptr) {
              v = f32_to_bf16(bf16_to_f32(v) + bf16_to_f32(bias[out0 + rr]));
            }
            if (res != nullptr) {
              v = f32_to_bf16(bf16_to_f32(res[at]) + bf16_to_f32(v));
            }
            y[at] = v;
          } else {
            partial[static_cast<size_t>(blockIdx.y) * M_all * N + at] = acc[c][i];
          }
        }
      }
    }
  }
}

// ---- stream tile ---------------------------------------------------------------------------
// The tile for chunks of 8..32 columns in whole 16-byte vectors (gemm_stream64 further down is
// its form for exactly 64): a workgroup of sixteen wavefronts owns 32 or 64 rows and all of K,
// or a share of K in whole chunks (grid.y) whose partials the last workgroup of a row block to
// finish adds up -- either way a launch has no second kernel; the epilogue is the reduce's
// (bias, residual, one rounding to bf16).  Eight of the wavefronts multiply, the other eight
// stage the operands into LDS; a barrier per chunk keeps the two sides one chunk apart.  (One
// set of wavefronts doing both took the sum of the two times per chunk, 0.7 us at N = 8 and
// 1.2 us at N = 32 on 7168x5120; two sets take the longer one.)
//
// Weights never become bf16(level * scale).  A packed byte goes through a pair table (byte ->
// the two levels as a bf16 pair, one conflict-free LDS read) and the four pairs of a dword are
// an MFMA A operand as they are.  The k-to-slot map keeps every MFMA inside one 64-wide group:
// lane l of v_mfma_f32_32x32x16_bf16 supplies eight k of row l % 32 in slots 8 (l / 32) .. + 8,
// a wavefront step is one group, lane l takes the sixteen bytes (32 codes) of row l % 32 at
// byte 16 (l / 32) of the group, and the step's four MFMAs take its four dwords: k =
// 32 (l / 32) + 8 j .. + 8.  Their sum over the group starts from zero and enters the
// accumulator through one fp32 multiply-add with the group's scale per output row, so the
// scale is applied once per 64 products instead of once per weight, exactly (fp16 -> fp32),
// and the only rounding of a weight is bf16(level).
//
// K is walked in chunks of 512 (eight groups): multiplying wavefront w works on group w of
// every chunk, all eight on the same rows (with 64 rows a workgroup every B operand it reads
// feeds two A operands), and their eight sums of an output meet in LDS at the end, added in
// the order of the wavefronts.  Every element of x is therefore read from LDS once per
// workgroup, and every B operand by one wavefront only.
//
// Scales: all of the rows' scales are staged in LDS at the start ([group][row], fp16).  An
// accumulator lane holds rows 8 b + 4 (l / 32) + i (b, i = 0..3) of a 32-row block: lane l
// reads the scale of row 8 ((l % 16) / 4) + 4 (l / 32) + l % 4, which puts the row of
// accumulator value v at position v of every row of sixteen lanes, where a DPP row broadcast
// fetches it.
//
// Global memory is read with consecutive lanes on consecutive bytes only (a load whose lanes
// read 64 different rows keeps the memory pipeline's address stage busy for some 140 cycles
// whatever its width, and the MFMA layout is one row per lane): a chunk of weights, 32 rows x
// 256 bytes, is one 16-byte load per staging thread, passed through LDS (row stride 272
// bytes, conflict-free for the 16-byte operand reads); a chunk of x is one or two items per
// staging thread (two k x eight columns each), or at 32 columns four whole-line pieces,
// interleaved into the transposed chunk buffer.
//
// Pipeline: a staging thread keeps its loads of kStreamRing chunks in
// flight in registers and stores a chunk to LDS (two buffers) one chunk ahead of its use.
// Every request is unconditional -- past the end of K it repeats the last chunk, unused --
// and the chunks of a workgroup (at most kStreamBodies) are written out nested, chunk c + 1
// inside the "if" of chunk c, instead of looped over, because vector loads return in order
// and are waited for by count: only with a fixed number of requests between a request and its
// use can the compiler wait for the oldest alone, and where a loop closes, or two paths meet,
// its count starts over (it waits there for nearly everything in flight, and the ring needs
// as many chunks again to fill).

// The pair table of this tile: entry (byte, copy) at byte * 128 + copy * 4, 32 copies.  The
// LDS serves a 4-byte read of a wavefront in two halves of 32 lanes, so lane & 31 picking the
// copy keeps the lookups free of bank conflicts in 32 KB instead of the GEMV's 64 KB (measured:
// the same conflict count and the same time); the address costs a shift and an and-or instead
// of one v_perm_b32.  Filled by sixteen wavefronts: wavefront v writes the bytes whose low
// code is v, lanes 0..31 / 32..63 the even / odd high codes.
__device__ __forceinline__ void fill_pair_table32(uint32_t *table, int wave16, int lane) {
  const uint32_t lo = bf16_bits_rne(kLutBits[wave16]);
  const int copy = lane & 31, half = lane >> 5;
#pragma unroll
  for (int jj = 0; jj < 8; ++jj) {
    const int j = 2 * jj + half;
    const uint32_t hi = (half ? bf16_bits_rne(kLevelBits[2 * jj + 1]) : bf16_bits_rne(kLevelBits[2 * jj])) << 16;
    table[((wave16 + 16 * j) << 5) + copy] = lo | hi;
  }
}
// the pair of byte J of w; copy4 = 4 * (lane & 31)
template <int J>
__device__ __forceinline__ uint32_t pair32_at(uint32_t w, uint32_t copy4) {
  const uint32_t sh = J == 0 ? (w << 7) : (w >> (8 * J - 7));
  return lds0_u32((sh & 0x7F80u) | copy4);
}

// f(0); if (1 < n) { f(1); if (2 < n) { ... } }: chunk C is reached through chunk C - 1 only, so
// the compiler knows every request of the earlier chunks to have been issued.
template <int C, int MAX, class F>
__device__ __forceinline__ void nest_chunks(int n, F &f) {
  if constexpr (C < MAX) {
    if (C == 0 || C < n) {
      f(std::integral_constant<int, C>{});
      nest_chunks<C + 1, MAX>(n, f);
    }
  }
}

// acc[v] += (position v of this lane's row of sixteen lanes of `mine`) * t[v] for the sixteen
// values of a 32x32 result, one v_fmac_f32_dpp each (the compiler keeps the broadcast and the
// multiply-add apart), written as two statements of eight so that nothing the compiler emits
// can stand where a hazard would be:
//  - the matrix core's result registers may be read by hand-written instructions only after it
//    has finished writing them (up to 18 wait states after the last MFMA was issued); the
//    compiler counts those for its own instructions, not for what an asm statement reads: the
//    first statement opens with the wait states, and t goes through it as a whole;
//  - a DPP operand must have been written two instructions or more before it is read, and the
//    compiler may compute or copy an asm operand right in front of the statement (seen once: a
//    stale value in accumulator 0 of every block): both statements open with wait states for
//    that too.
#define CHR_FMAC8(FIRST)                                                                  \
  "v_fmac_f32_dpp %0, %16, %8 row_newbcast:" #FIRST "+0 row_mask:0xf bank_mask:0xf\n\t"    \
  "v_fmac_f32_dpp %1, %16, %9 row_newbcast:" #FIRST "+1 row_mask:0xf bank_mask:0xf\n\t"    \
  "v_fmac_f32_dpp %2, %16, %10 row_newbcast:" #FIRST "+2 row_mask:0xf bank_mask:0xf\n\t"   \
  "v_fmac_f32_dpp %3, %16, %11 row_newbcast:" #FIRST "+3 row_mask:0xf bank_mask:0xf\n\t"   \
  "v_fmac_f32_dpp %4, %16, %12 row_newbcast:" #FIRST "+4 row_mask:0xf bank_mask:0xf\n\t"   \
  "v_fmac_f32_dpp %5, %16, %13 row_newbcast:" #FIRST "+5 row_mask:0xf bank_mask:0xf\n\t"   \
  "v_fmac_f32_dpp %6, %16, %14 row_newbcast:" #FIRST "+6 row_mask:0xf bank_mask:0xf\n\t"   \
  "v_fmac_f32_dpp %7, %16, %15 row_newbcast:" #FIRST "+7 row_mask:0xf bank_mask:0xf"
__device__ __forceinline__ void scale_into_all(f32x16 &acc, float mine, const f32x16 &t) {
  float a[16], v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    a[i] = acc[i];
    v[i] = t[i];
  }
  asm volatile("s_nop 15\n\ts_nop 7\n\t" CHR_FMAC8(0)
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
               : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(mine));
  asm volatile("s_nop 1\n\t" CHR_FMAC8(8)
               : "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]),
                 "+v"(a[15])
               : "v"(v[8]), "v"(v[9]), "v"(v[10]), "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]),
                 "v"(mine));
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc[i] = a[i];
  }
}
#undef CHR_FMAC8

// The low halves of a and b as one dword, a below b; the high halves likewise: a byte
// permute each.
__device__ __forceinline__ uint32_t low_halves(uint32_t a, uint32_t b) {
  return __builtin_amdgcn_perm(b, a, 0x05040100u);
}
__device__ __forceinline__ uint32_t high_halves(uint32_t a, uint32_t b) {
  return __builtin_amdgcn_perm(b, a, 0x07060302u);
}

// `own` in the lanes of the banks (fours of a row of sixteen lanes) that MASK leaves out, what
// the DPP pattern CTRL brings of `other` in the rest.
template <int CTRL, int MASK>
__device__ __forceinline__ uint32_t dpp_into(uint32_t own, uint32_t other) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(own), static_cast<int>(other),
                                                           CTRL, 0xF, MASK, false));
}

// Row of a chunk buffer that holds token n.  A staging instruction of 17..32 columns stores
// tokens 8 q + e for all four vectors q and sixteen consecutive k pairs: with the tokens in
// order, a token row being 260 dwords = 4 banks on, vectors q and q + 2 would meet in the
// same banks.  The order below puts the four vectors of an instruction 16 banks apart and
// still keeps tokens 0..15, and 16..31, in sixteen rows of different banks for the operand
// reads.  Up to 16 columns (two vectors x 32 k pairs an instruction) the plain order is the
// one without conflicts.
template <int XI>
__device__ __forceinline__ int stream_token_row(int n) {
  if constexpr (XI != 2) {
    return n;
  } else {
    const int q = n >> 3, e = n & 7;
    return (n & 16) + ((4 * q + (e & 3) + 8 * (e >> 2)) & 15);
  }
}

// XI: how a staging thread fetches x: one item (two k x eight columns) up to 16 columns, two
// above, four quarter items at exactly 32 columns.  RB: 32-row blocks of a workgroup, 1 or 2
// (segs.blocks counts blocks of 32 RB rows): with two, a multiplying wavefront feeds every B
// operand it reads to two A operands, and x is staged once per 64 rows.
// Arrival counts of the stream tile's K splits, one word a row block: the workgroup that finds
// the others of its row block already counted adds up the partials.  All zero when the library
// is loaded, and every launch leaves them zero.  A launch uses one slot; launches that may
// overlap in time must use different slots (the host deals a slot to every stream).
static __device__ unsigned int stream_arrivals[kArriveSlots][kArriveBlocks];

// PAIR (with two row blocks): they are rows 32 b .. + 32 of two matrices of the same shape,
// gate (segs' first) and up (second), and the epilogue stores silu(gate) * up, [M, N], with
// reduce_swiglu's roundings: no partials and no reduce launch.  grid.y must be 1.
template <int XI, int RB, bool PAIR = false>
__global__ __launch_bounds__(kStreamBlock) void gemm_stream(const GemmSegs segs,
                                                            const uint16_t *__restrict__ x,
                                                            uint16_t *__restrict__ y,
                                                            float *__restrict__ partial, int M_all,
                                                            int K, int K_pad, int N,
                                                            const uint16_t *__restrict__ bias,
                                                            const uint16_t *res, int arrive_slot,
                                                            float *__restrict__ colsq) {
  constexpr int XS = kStreamXS;
  constexpr int CK = kStreamChunkK;
  constexpr int ROWS = kStreamRows * RB;
  constexpr uint32_t kWBuf = RB * kStreamWBytes;
  constexpr uint32_t kXAddr = kStreamTableBytes;
  constexpr uint32_t kWAddr = kXAddr + 2 * kStreamXBytes;
  constexpr uint32_t kScaleAddr = kWAddr + 2 * kWBuf;
  static_assert(kScaleAddr + stream_scale_bytes(RB) == stream_lds_bytes(RB), "LDS map");
  static_assert(8 * 64 * 16 * RB * 4 <= kWAddr, "the wavefronts' sums reuse the table and x");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave16 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool stager = wave16 >= 8;  // wavefronts 8..15 stage, 0..7 multiply
  const int wave = wave16 & 7;      // group of a chunk (multiplying), or eighth of the staging
  const int stid = tid & (kStreamStagers - 1);
  static_assert(!PAIR || RB == 2, "a pair is two row blocks");
  int bx = static_cast<int>(blockIdx.x);
  int seg = 0;
  if constexpr (!PAIR) {
    if (bx >= segs.blocks[0]) {
      bx -= segs.blocks[0];
      seg = 1;
      if (bx >= segs.blocks[1]) {
        bx -= segs.blocks[1];
        seg = 2;
      }
    }
  }
  const uint8_t *__restrict__ packed = segs.packed[seg];
  const uint16_t *__restrict__ scale = segs.scale[seg];
  const int M = segs.M[seg];
  const int out0 = segs.row0[seg];
  const int row_base = bx * (PAIR ? kStreamRows : ROWS);  // first row, of each matrix when PAIR
  const int r = lane & 31;  // row of the A operand, token of the B operand
  const int h = lane >> 5;  // which half of a group's k
  // grid.y splits K by whole chunks: this workgroup takes n_ch of them from chunk c0 on, and
  // from here on x, K, row_bytes and groups describe what is left of K from that chunk on
  const int n_ch_all = (K_pad + CK - 1) / CK;
  const int per_split = segs.per_split;
  const unsigned int n_splits = static_cast<unsigned int>(segs.splits);
  const int c0 = static_cast<int>(blockIdx.y) * per_split;
  const int n_ch = min(per_split, n_ch_all - c0);
  const int row_stride = K_pad >> 1;  // bytes of a packed row
  const int row_bytes = row_stride - c0 * (CK / 2);
  const int groups_all = K_pad >> 6;
  const int groups = min(8 * n_ch, groups_all - 8 * c0);
  x += static_cast<size_t>(c0) * CK * N;
  K -= c0 * CK;

  // ---- requests: a thread's share of one chunk ------------------------------------------------
  // XI = 4 is the form for exactly 32 columns: a k pair of x (rows 2 kp, 2 kp + 1) is then
  // one 128-byte line, which eight consecutive lanes fetch 16 bytes each -- 1 KB of whole
  // lines per load instruction -- and the lanes that hold the same columns of the two rows
  // (j and 7 - j of the eight) swap halves through a DPP half-row mirror before they
  // interleave: four loads a thread and chunk, each a quarter of an item of the other forms.
  constexpr bool WIDE = XI == 4;
  constexpr int NA = WIDE ? 4 : XI, NB = WIDE ? 0 : XI;
  // a thread's loads of one chunk: w = bytes 16 (stid % 16) .. + 16 of the chunk of row
  // stid / 16; a, b = x, rows 2 kp and 2 kp + 1 of the chunk, columns 8 q .. + 8
  struct Item {
    uint4 a[NA], b[NB > 0 ? NB : 1];
  };
  const int w_piece = 16 * (stid & 15);
  const int nv = N >> 3;
  const int n_items = (CK / 2) * nv;
  int xkp[NA], xq[NA];
#pragma unroll
  for (int it = 0; it < NA; ++it) {
    const int idx = min(stid + it * kStreamStagers, n_items - 1);
    xkp[it] = idx / nv;
    xq[it] = idx - xkp[it] * nv;
  }
  // the wide form: lane j of eight holds row 2 kp + (j >> 2), columns 8 q with q = j or 7 - j
  const int w_half = (lane >> 2) & 1;
  const int w_q = w_half ? 7 - (lane & 7) : (lane & 7);
  const int w_kp = (lane >> 3) + 8 * wave;  // + 64 it
  // Requests take a base that is the same in every lane (it moves from chunk to chunk on the
  // scalar side) and a 32-bit offset of the lane: what does not depend on the chunk is in
  // registers, and a request costs the clamp that keeps the tail of K inside x and the row.
  uint32_t w_off[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    w_off[rb] = static_cast<uint32_t>(min(row_base + (PAIR ? 0 : 32 * rb) + (stid >> 4), M - 1)) * row_stride +
                c0 * (CK / 2);
  }
  const uint32_t x_row = 2u * N;  // bytes of a row of x
  uint32_t xk_off[NA], xq_off[NA];
#pragma unroll
  for (int it = 0; it < NA; ++it) {
    xk_off[it] = WIDE ? (2 * (w_kp + 64 * it) + w_half) * x_row : 2 * xkp[it] * x_row;
    xq_off[it] = 16u * (WIDE ? w_q : xq[it]);
  }
  auto load = [&](int c, U32x4 &w0, U32x4 &w1, Item &v) {
    const int cc = min(c, n_ch - 1);
    const uint32_t w_at = min(static_cast<uint32_t>(cc * (CK / 2) + w_piece), static_cast<uint32_t>(row_bytes - 16));
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      (rb ? w1 : w0) =
          *reinterpret_cast<const U32x4 *>((PAIR && rb ? segs.packed[1] : packed) + (w_off[rb] + w_at));
    }
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x) + static_cast<size_t>(cc) * CK * x_row;
    const uint32_t k_last = static_cast<uint32_t>(K - 1 - cc * CK) * x_row;  // offset of the last row of x
#pragma unroll
    for (int it = 0; it < NA; ++it) {
      v.a[it] = *reinterpret_cast<const uint4 *>(xb + (min(xk_off[it], k_last) + xq_off[it]));
      if constexpr (!WIDE) {
        v.b[it] = *reinterpret_cast<const uint4 *>(xb + (min(xk_off[it] + x_row, k_last) + xq_off[it]));
      }
    }
  };
  auto store = [&](int c, const U32x4 w0, const U32x4 w1, const Item &v) {
    const int buf = c & 1;
    // weights: row-major, 272 bytes a row.  A piece past the end of the row (the second half
    // of a last chunk of 256) repeats the row's last 16 bytes; x is zero there.
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      *reinterpret_cast<U32x4 *>(lds_raw + kWAddr + buf * kWBuf + (32 * rb + (stid >> 4)) * kStreamWStride +
                                 w_piece) = rb ? w1 : w0;
    }
    uint32_t *xd = reinterpret_cast<uint32_t *>(lds_raw + kXAddr + buf * kStreamXBytes);
    const bool tail = (c + 1) * CK > K;  // only the chunk at the end of K has rows of x to blank
    if constexpr (WIDE) {
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int kp = w_kp + 64 * it;
        uint32_t m0 = v.a[it].x, m1 = v.a[it].y, m2 = v.a[it].z, m3 = v.a[it].w;
        if (tail) {
          asm volatile("" ::: "memory");  // (a branch, not four selects in every chunk)
          const bool live = c * CK + 2 * kp + w_half < K;
          m0 = live ? m0 : 0u;
          m1 = live ? m1 : 0u;
          m2 = live ? m2 : 0u;
          m3 = live ? m3 : 0u;
        }
        // Lanes 0..3 of eight hold the even row of a k pair, lanes 4..7 the odd one, mirrored:
        // partners hold the same eight tokens.  The even row's lane makes tokens 8 q .. + 4
        // (a = its own tokens 0..3, b = the partner's), the odd row's lane tokens 8 q + 4 ..
        // + 4 (a = the partner's tokens 4..7, b = its own): the half-row mirror brings the
        // partner's dwords into the lanes of banks 1 and 3 (odd rows), or 0 and 2.
        const uint32_t a0 = dpp_into<0x141, 0xA>(m0, m2), a1 = dpp_into<0x141, 0xA>(m1, m3);
        const uint32_t b0 = dpp_into<0x141, 0x5>(m2, m0), b1 = dpp_into<0x141, 0x5>(m3, m1);
        // token 4 u + e lives in row 8 e + u of the chunk buffer: the eight lanes of a k pair
        // (u = 2 q + half) store into eight consecutive rows, 4 banks apart, and the four k
        // pairs of 32 lanes fill the banks between -- no two lanes on a bank, where rows in
        // token order (eight rows 4 apart, 16 banks apart) put four there
        uint32_t *dst = xd + (2 * w_q + w_half) * (XS / 2) + kp;
        dst[0] = low_halves(a0, b0);
        dst[8 * (XS / 2)] = high_halves(a0, b0);
        dst[16 * (XS / 2)] = low_halves(a1, b1);
        dst[24 * (XS / 2)] = high_halves(a1, b1);
      }
    } else {
#pragma unroll
      for (int it = 0; it < NB; ++it) {
        if (stid + it * kStreamStagers < n_items) {
          uint32_t a[4] = {v.a[it].x, v.a[it].y, v.a[it].z, v.a[it].w};
          uint32_t b[4] = {v.b[it].x, v.b[it].y, v.b[it].z, v.b[it].w};
          if (tail) {
            asm volatile("" ::: "memory");  // (a branch, not eight selects in every chunk)
            const int k = c * CK + 2 * xkp[it];
            const bool ka = k < K, kb = k + 1 < K;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              a[e] = ka ? a[e] : 0u;
              b[e] = kb ? b[e] : 0u;
            }
          }
          uint32_t *dst = xd + xkp[it];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            dst[stream_token_row<XI>(8 * xq[it] + 2 * e) * (XS / 2)] = low_halves(a[e], b[e]);
            dst[stream_token_row<XI>(8 * xq[it] + 2 * e + 1) * (XS / 2)] = high_halves(a[e], b[e]);
          }
        }
      }
    }
  };

  // ---- set-up -------------------------------------------------------------------------------
  // The rows' scales (four groups -- 8 aligned bytes, K_pad being a multiple of 256 -- a
  // request, a fixed number of requests a thread, the surplus repeating the last one) and
  // the staging wavefronts' requests in the order the chunks keep them in; the table while
  // they travel.
  constexpr int kScaleLoads = (ROWS * (kStreamMaxGroups / 4) + kStreamBlock - 1) / kStreamBlock;
  const int quads = groups >> 2;
  uint2 sv[kScaleLoads];
#pragma unroll
  for (int it = 0; it < kScaleLoads; ++it) {
    const int i = min(tid + it * kStreamBlock, ROWS * quads - 1);
    const int srow = i / quads;
    const uint16_t *sc = PAIR && srow >= 32 ? segs.scale[1] : scale;
    sv[it] = *reinterpret_cast<const uint2 *>(
        sc + static_cast<size_t>(min(row_base + (PAIR ? srow & 31 : srow), M - 1)) * groups_all + 8 * c0 +
        4 * (i - srow * quads));
  }
  // chunks a staging thread keeps in flight (kStreamRing: deeper rings measured slower in every
  // form)
  constexpr int R = kStreamRing;
  Item ring[R];
  // (native vectors: the struct type's assignment would pin them in memory; the second block's
  // are idle with one block)
  U32x4 ring_w[R], ring_w1[R];
  if (stager) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      load(j, ring_w[j], ring_w1[j], ring[j]);
    }
  }
  fill_pair_table32(reinterpret_cast<uint32_t *>(lds_raw), wave16, lane);
  {
    // the rows of tokens N .. 32 of the chunk buffers are never staged: zero them once
    const int nz = (32 - N) * (XS / 2);
    for (int b = 0; b < 2; ++b) {
      uint32_t *z = reinterpret_cast<uint32_t *>(lds_raw + kXAddr + b * kStreamXBytes);
      for (int i = tid; i < nz; i += kStreamBlock) {
        const int n = N + i / (XS / 2);
        z[stream_token_row<XI>(n) * (XS / 2) + (i - (n - N) * (XS / 2))] = 0u;
      }
    }
  }
  {
    uint16_t *sl = reinterpret_cast<uint16_t *>(lds_raw + kScaleAddr);  // [group][row of the block]
#pragma unroll
    for (int it = 0; it < kScaleLoads; ++it) {
      const int i = tid + it * kStreamBlock;
      if (i < ROWS * quads) {
        const int srow = i / quads;
        const int gq = i - srow * quads;
        sl[(4 * gq + 0) * ROWS + srow] = static_cast<uint16_t>(sv[it].x);
        sl[(4 * gq + 1) * ROWS + srow] = static_cast<uint16_t>(sv[it].x >> 16);
        sl[(4 * gq + 2) * ROWS + srow] = static_cast<uint16_t>(sv[it].y);
        sl[(4 * gq + 3) * ROWS + srow] = static_cast<uint16_t>(sv[it].y >> 16);
      }
    }
  }
  if (stager) {
    store(0, ring_w[0], ring_w1[0], ring[0]);
    load(R, ring_w[0], ring_w1[0], ring[0]);
  }
  __syncthreads();

  // ---- the chunks: one barrier each, in both roles ------------------------------------------
  // (the multiplying wavefronts' sums live and die inside their branch, so that the staging
  // wavefronts' registers hold the ring alone)
  float *sums = reinterpret_cast<float *>(lds_raw);
  if (stager) {
    {
      auto chunk = [&](auto index) {
        constexpr int c = decltype(index)::value;
        constexpr int j = c % R;
        // chunk c + 1 goes into the buffers that chunk c - 1 was read from (the multiplying
        // wavefronts are past those reads: the barrier of chunk c - 1); its registers take
        // chunk c + 1 + R
        if (c + 1 < n_ch) {
          store(c + 1, ring_w[(j + 1) % R], ring_w1[(j + 1) % R], ring[(j + 1) % R]);
        }
        load(c + 1 + R, ring_w[(j + 1) % R], ring_w1[(j + 1) % R], ring[(j + 1) % R]);
        __syncthreads();
      };
      nest_chunks<0, kStreamBodies>(n_ch, chunk);
    }
  }
  // (a second question of its own, not an else: the staging wavefronts' ring is then dead
  // before the multiplying wavefronts' sums are born, and the two roles share registers)
  int role;
  asm volatile("s_mov_b32 %0, %1" : "=s"(role) : "s"(wave16));
  if (role < 8) {
    f32x16 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[rb][v] = 0.f;
      }
    }
    const uint32_t copy4 = static_cast<uint32_t>(lane & 31) << 2;
    const uint32_t x_lane =
        kXAddr + static_cast<uint32_t>(stream_token_row<XI>(r) * XS + 32 * h + 64 * wave) * 2;
    const uint32_t w_lane = kWAddr + static_cast<uint32_t>(r * kStreamWStride + 32 * wave + 16 * h);
    // this lane's scale: row 8 ((l % 16) / 4) + 4 h + l % 4 of the 32, group `wave` of the chunk
    const uint32_t s_lane =
        kScaleAddr + static_cast<uint32_t>(wave * ROWS + 8 * ((lane & 15) >> 2) + 4 * h + (lane & 3)) * 2;
    for (int c = 0; c < n_ch; ++c) {
      const uint32_t buf = static_cast<uint32_t>(c & 1);
      // a group past the end of K (last chunk of 256) multiplies zeros of x; its scale is read
      // from the last group that exists
      const int grp = min(8 * c + wave, groups - 1) - wave;
      float mine[RB];
      uint32_t w4[RB][4];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        mine[rb] = f16_to_f32(*reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(
            s_lane + static_cast<uint32_t>((grp * ROWS + 32 * rb) * 2)));
        const uint4 wv = lds0_u128(w_lane + buf * kWBuf + rb * kStreamWBytes);
        w4[rb][0] = wv.x;
        w4[rb][1] = wv.y;
        w4[rb][2] = wv.z;
        w4[rb][3] = wv.w;
      }
      const uint32_t xl = x_lane + buf * kStreamXBytes;
      f32x16 t[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          t[rb][v] = 0.f;
        }
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const uint4 b = lds0_u128(xl + 16 * jj);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const uint32_t w = w4[rb][jj];
          const uint4 a = make_uint4(pair32_at<0>(w, copy4), pair32_at<1>(w, copy4), pair32_at<2>(w, copy4),
                                     pair32_at<3>(w, copy4));
          t[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                          __builtin_bit_cast(bf16x8, b), t[rb], 0, 0, 0);
        }
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        scale_into_all(acc[rb], mine[rb], t[rb]);
      }
      __syncthreads();
    }
    // ---- the eight sums of every output meet in LDS -------------------------------------------
    // (the last barrier above has every wavefront past its reads of the table and of x)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        sums[((rb * 8 + wave) * 16 + v) * kWave + lane] = acc[rb][v];
      }
    }
  }
  __syncthreads();
  // wavefront w of the sixteen finishes accumulator value w of every 32-row block
  float o32[RB];
  size_t at[RB];
  bool live[RB];
  int orow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int v = wave16;
    o32[rb] = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      o32[rb] += sums[((rb * 8 + q) * 16 + v) * kWave + lane];
    }
    const int rr = row_base + (PAIR ? 0 : 32 * rb) + 8 * (v >> 2) + 4 * h + (v & 3);
    live[rb] = r < N && rr < M;
    orow[rb] = out0 + min(rr, M - 1);
    // (at 32 columns row r of the chunk buffers, the B operand's column r, holds token
    // 4 (r % 8) + r / 8)
    at[rb] = static_cast<size_t>(orow[rb]) * N + (WIDE ? 4 * (r & 7) + (r >> 3) : min(r, N - 1));
  }
  if constexpr (PAIR) {
    // output 0 is the gate's, output 1 the up's, at the same row and token
    if (live[0]) {
      const float a = bf16_to_f32(f32_to_bf16(o32[0]));
      const float act = bf16_to_f32(f32_to_bf16(a / (1.f + expf(-a))));
      y[at[0]] = f32_to_bf16(act * bf16_to_f32(f32_to_bf16(o32[1])));
    }
    return;
  }
  if (partial != nullptr) {
    // this split's slab of the partials
    const size_t slab = static_cast<size_t>(M_all) * N;
    if (arrive_slot < 0) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (live[rb]) {
          partial[blockIdx.y * slab + at[rb]] = o32[rb];
        }
      }
      return;  // a reduce kernel adds the slabs up
    }
    // The last of this row block's splits to arrive adds them up, in split order whoever it
    // is; nobody waits for anybody.  The compute dies' L2 caches do not see each other's
    // lines, and a fence that makes them (write back and invalidate the whole cache) costs
    // tens of microseconds with a few hundred workgroups at it.  So the partials and the
    // count go past the caches one access at a time instead: device-scope stores that write
    // through, waited for by every thread before the barrier after which thread 0 counts the
    // workgroup in, and device-scope loads that do not take a cached line for an answer.
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (live[rb]) {
        __hip_atomic_store(partial + blockIdx.y * slab + at[rb], o32[rb], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int *last = reinterpret_cast<int *>(lds_raw + kScaleAddr);  // (the scales are done with)
    if (tid == 0) {
      unsigned int *count = &stream_arrivals[arrive_slot][blockIdx.x];
      const unsigned int before =
          __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool all_in = before + 1 == n_splits;
      if (all_in) {
        __hip_atomic_store(count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      *last = all_in ? 1 : 0;
    }
    __syncthreads();
    if (*last == 0) {
      return;
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      // (four requests at a time: a loop of single ones waits a round trip for each)
      float sum = 0.f;
      for (unsigned int j0 = 0; j0 < n_splits; j0 += 4) {
        float v[4];
#pragma unroll
        for (unsigned int u = 0; u < 4; ++u) {
          v[u] = __hip_atomic_load(partial + min(j0 + u, n_splits - 1) * slab + at[rb], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (unsigned int u = 0; u < 4; ++u) {
          sum = j0 + u == 0 ? v[0] : (j0 + u < n_splits ? sum + v[u] : sum);
        }
      }
      o32[rb] = sum;
    }
  }
  float square[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    square[rb] = 0.f;
    if (live[rb]) {
      // the epilogue of reduce_splitk, here (res may alias y: same thread, same element)
      uint16_t o = f32_to_bf16(o32[rb]);
      if (bias != nullptr) {
        o = f32_to_bf16(bf16_to_f32(o) + bf16_to_f32(bias[orow[rb]]));
      }
      if (res != nullptr) {
        o = f32_to_bf16(bf16_to_f32(res[at[rb]]) + bf16_to_f32(o));
      }
      y[at[rb]] = o;
      square[rb] = bf16_to_f32(o) * bf16_to_f32(o);
    }
  }
  if constexpr (WIDE) {
    // What reduce_splitk_sq leaves for the RMSNorm that reads y next, here: the column sums
    // of squares of the values as stored, per block of 1024 / 32 = 32 rows -- a 32-row block
    // of this workgroup, whose 32 contributions to a column (sixteen wavefronts, two lanes)
    // meet in LDS and are added in a fixed order.  One matrix only (rows from 0).
    if (colsq != nullptr) {
      __syncthreads();  // every wavefront is past its reads of `sums`
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        sums[(rb * 16 + wave16) * kWave + lane] = square[rb];
      }
      __syncthreads();
      if (tid < 32 * RB) {
        const int b = tid >> 5, col = tid & 31;
        const int rcol = (col >> 2) + 8 * (col & 3);  // the B operand's column that holds token col
        float sum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          sum += sums[(b * 16 + v) * kWave + rcol];
          sum += sums[(b * 16 + v) * kWave + rcol + 32];
        }
        if (row_base + 32 * b < M) {
          colsq[static_cast<size_t>((row_base >> 5) + b) * 32 + col] = sum;
        }
      }
    }
  }
}

// ---- the same tile for chunks of exactly 64 columns -------------------------------------------
// Two 32-column B operands per A operand: what a wavefront looks up once multiplies 64 tokens.
// A workgroup owns 64 rows; K is walked in chunks of 256 (four groups), multiplying wavefront
// w takes group w % 4 of row block w / 4 and both halves of the tokens, so every weight goes
// through the table once per workgroup and every element of x is read from LDS by two
// wavefronts.  A row of x is then exactly one 128-byte line: eight lanes fetch it 16 bytes
// each, the next eight the row after it, and lanes eight apart (same tokens, rows k and
// k + 1) swap halves through a DPP rotation of their row of sixteen before they interleave.
// The chunk buffers hold the tokens in an order that spreads those stores over the banks
// (the B operand's column l of block cb is token 4 (l % 16) + 2 cb + l / 16).
// Everything else -- the pair table, the scales in LDS and their DPP broadcast, the ring of
// requests and the nested chunks, the splits of K that meet in the tile -- is gemm_stream's.
// PAIR: the two 32-row blocks of a workgroup are rows 32 b .. + 32 of two matrices of the same
// shape, gate (segs' first) and up (second), and the epilogue stores silu(gate) * up, [M, 64],
// with reduce_swiglu's roundings: no partials and no reduce launch.  grid.y must be 1.
template <bool PAIR>
__global__ __launch_bounds__(kStreamBlock) void gemm_stream64(GemmSegs segs,
                                                              const uint16_t *__restrict__ x,
                                                              uint16_t *__restrict__ y,
                                                              float *__restrict__ partial, int M_all,
                                                              int K, int K_pad,
                                                              const uint16_t *__restrict__ bias,
                                                              const uint16_t *res, int arrive_slot,
                                                              float *__restrict__ colsq) {
  constexpr int XS = kWideXS;
  constexpr int CK = kWideChunkK;
  constexpr int ROWS = kWideRows;
  constexpr int N = 64;
  constexpr uint32_t kXAddr = kStreamTableBytes;
  constexpr uint32_t kWAddr = kXAddr + 2 * kWideXBytes;
  constexpr uint32_t kScaleAddr = kWAddr + 2 * kWideWBytes;
  static_assert(kScaleAddr + kWideScaleBytes == kWideLdsBytes, "LDS map");
  static_assert(8 * 2 * 16 * 64 * 4 <= kWAddr, "the wavefronts' sums reuse the table and x");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave16 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool stager = wave16 >= 8;  // wavefronts 8..15 stage, 0..7 multiply
  const int wave = wave16 & 7;
  const int stid = tid & (kStreamStagers - 1);
  int bx = static_cast<int>(blockIdx.x);
  int seg = 0;
  if constexpr (!PAIR) {
    if (bx >= segs.blocks[0]) {
      bx -= segs.blocks[0];
      seg = 1;
      if (bx >= segs.blocks[1]) {
        bx -= segs.blocks[1];
        seg = 2;
      }
    }
  }
  // (PAIR: the staging wavefronts 8..11 fetch gate rows, 12..15 up rows)
  const uint8_t *__restrict__ packed = segs.packed[PAIR ? (wave16 >= 12 ? 1 : 0) : seg];
  const uint16_t *__restrict__ scale = segs.scale[seg];
  const int M = segs.M[seg];
  const int out0 = segs.row0[seg];
  const int row_base = bx * (PAIR ? 32 : ROWS);  // first row, of each matrix when PAIR
  const int r = lane & 31;  // row of the A operand, token of the B operand
  const int h = lane >> 5;  // which half of a group's k
  // grid.y splits K by whole chunks (see gemm_stream): from here on x, K, row_bytes and groups
  // describe what is left of K from this workgroup's first chunk on
  const int n_ch_all = (K_pad + CK - 1) / CK;
  const int per_split = segs.per_split;
  const unsigned int n_splits = static_cast<unsigned int>(segs.splits);
  const int c0 = static_cast<int>(blockIdx.y) * per_split;
  const int n_ch = min(per_split, n_ch_all - c0);
  const int row_stride = K_pad >> 1;
  const int row_bytes = row_stride - c0 * (CK / 2);
  const int groups_all = K_pad >> 6;
  const int groups = min(4 * n_ch, groups_all - 4 * c0);
  x += static_cast<size_t>(c0) * CK * N;
  K -= c0 * CK;

  // ---- requests: a thread's share of one chunk ------------------------------------------------
  // w = bytes 16 (stid % 8) .. + 16 of the chunk of row stid / 8 (a row's 128 bytes of a chunk
  // are one line); a[it] = x, row 2 kp + half of the chunk, tokens 8 q .. + 8, with kp =
  // lane / 16 + 4 wave + 32 it, half = (lane / 8) % 2, q = lane % 8
  struct Item {
    uint4 a[4];
  };
  const int w_piece = 16 * (stid & 7);
  // (a base that is the same in every lane and a 32-bit offset of the lane: see gemm_stream)
  const uint32_t w_off =
      static_cast<uint32_t>(min(row_base + (PAIR ? (stid >> 3) & 31 : stid >> 3), M - 1)) * row_stride +
      c0 * (CK / 2);
  const int w_half = (lane >> 3) & 1;
  const int w_q = lane & 7;
  const int w_kp = (lane >> 4) + 4 * wave;  // + 32 it
  constexpr uint32_t x_row = 2u * N;  // bytes of a row of x
  uint32_t xk_off[4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    xk_off[it] = (2 * (w_kp + 32 * it) + w_half) * x_row;
  }
  const uint32_t xq_off = 16u * w_q;
  auto load = [&](int c, U32x4 &w, Item &v) {
    const int cc = min(c, n_ch - 1);
    const uint32_t w_at = min(static_cast<uint32_t>(cc * (CK / 2) + w_piece), static_cast<uint32_t>(row_bytes - 16));
    w = *reinterpret_cast<const U32x4 *>(packed + (w_off + w_at));
    const unsigned char *xb = reinterpret_cast<const unsigned char *>(x) + static_cast<size_t>(cc) * CK * x_row;
    const uint32_t k_last = static_cast<uint32_t>(K - 1 - cc * CK) * x_row;  // offset of the last row of x
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      v.a[it] = *reinterpret_cast<const uint4 *>(xb + (min(xk_off[it], k_last) + xq_off));
    }
  };
  auto store = [&](int c, const U32x4 w, const Item &v) {
    const int buf = c & 1;
    *reinterpret_cast<U32x4 *>(lds_raw + kWAddr + buf * kWideWBytes + (stid >> 3) * kWideWStride + w_piece) = w;
    uint32_t *xd = reinterpret_cast<uint32_t *>(lds_raw + kXAddr + buf * kWideXBytes);
    const bool tail = (c + 1) * CK > K;  // only the chunk at the end of K has rows of x to blank
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int kp = w_kp + 32 * it;
      uint32_t m0 = v.a[it].x, m1 = v.a[it].y, m2 = v.a[it].z, m3 = v.a[it].w;
      if (tail) {
        asm volatile("" ::: "memory");  // (a branch, not four selects in every chunk)
        const bool live = c * CK + 2 * kp + w_half < K;
        m0 = live ? m0 : 0u;
        m1 = live ? m1 : 0u;
        m2 = live ? m2 : 0u;
        m3 = live ? m3 : 0u;
      }
      // Lanes 0..7 of sixteen hold the even row of a k pair, lanes 8..15 the odd one, the same
      // tokens eight lanes apart.  The even row's lane makes tokens 8 q .. + 4 (a = its own
      // tokens 0..3, b = the partner's), the odd row's lane tokens 8 q + 4 .. + 4 (a = the
      // partner's tokens 4..7, b = its own): a rotation by eight brings the partner's dwords
      // into the lanes of banks 2 and 3 (odd rows), or 0 and 1.
      const uint32_t a0 = dpp_into<0x128, 0xC>(m0, m2), a1 = dpp_into<0x128, 0xC>(m1, m3);
      const uint32_t b0 = dpp_into<0x128, 0x3>(m2, m0), b1 = dpp_into<0x128, 0x3>(m3, m1);
      // token 4 u + e lives in row 16 e + u of the chunk buffer: the sixteen lanes of a k pair
      // (u = 2 q + half) then store into sixteen consecutive rows, 4 banks apart -- two lanes
      // a bank, where rows in token order (sixteen rows 4 apart, 16 banks apart) put eight
      // lanes on a bank
      uint32_t *dst = xd + (2 * w_q + w_half) * (XS / 2) + kp;
      dst[0] = low_halves(a0, b0);
      dst[16 * (XS / 2)] = high_halves(a0, b0);
      dst[32 * (XS / 2)] = low_halves(a1, b1);
      dst[48 * (XS / 2)] = high_halves(a1, b1);
    }
  };

  // ---- set-up -------------------------------------------------------------------------------
  constexpr int kScaleLoads = (ROWS * (kWideMaxGroups / 4) + kStreamBlock - 1) / kStreamBlock;
  const int quads = groups >> 2;
  uint2 sv[kScaleLoads];
#pragma unroll
  for (int it = 0; it < kScaleLoads; ++it) {
    const int i = min(tid + it * kStreamBlock, ROWS * quads - 1);
    const int srow = i / quads;
    const uint16_t *sc = PAIR && srow >= 32 ? segs.scale[1] : scale;
    sv[it] = *reinterpret_cast<const uint2 *>(
        sc + static_cast<size_t>(min(row_base + (PAIR ? srow & 31 : srow), M - 1)) * groups_all + 4 * c0 +
        4 * (i - srow * quads));
  }
  constexpr int R = kStreamRing;
  Item ring[R];
  U32x4 ring_w[R];
  if (stager) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      load(j, ring_w[j], ring[j]);
    }
  }
  fill_pair_table32(reinterpret_cast<uint32_t *>(lds_raw), wave16, lane);
  {
    uint16_t *sl = reinterpret_cast<uint16_t *>(lds_raw + kScaleAddr);  // [group][row of the block]
#pragma unroll
    for (int it = 0; it < kScaleLoads; ++it) {
      const int i = tid + it * kStreamBlock;
      if (i < ROWS * quads) {
        const int srow = i / quads;
        const int gq = i - srow * quads;
        sl[(4 * gq + 0) * ROWS + srow] = static_cast<uint16_t>(sv[it].x);
        sl[(4 * gq + 1) * ROWS + srow] = static_cast<uint16_t>(sv[it].x >> 16);
        sl[(4 * gq + 2) * ROWS + srow] = static_cast<uint16_t>(sv[it].y);
        sl[(4 * gq + 3) * ROWS + srow] = static_cast<uint16_t>(sv[it].y >> 16);
      }
    }
  }
  if (stager) {
    store(0, ring_w[0], ring[0]);
    load(R, ring_w[0], ring[0]);
  }
  __syncthreads();

  // ---- the chunks: one barrier each, in both roles (two questions, not an else: see
  // gemm_stream) ------------------------------------------------------------------------------
  float *sums = reinterpret_cast<float *>(lds_raw);
  if (stager) {
    auto chunk = [&](auto index) {
      constexpr int c = decltype(index)::value;
      constexpr int j = c % R;
      if (c + 1 < n_ch) {
        store(c + 1, ring_w[(j + 1) % R], ring[(j + 1) % R]);
      }
      load(c + 1 + R, ring_w[(j + 1) % R], ring[(j + 1) % R]);
      __syncthreads();
    };
    nest_chunks<0, kWideBodies>(n_ch, chunk);
  }
  int role;
  asm volatile("s_mov_b32 %0, %1" : "=s"(role) : "s"(wave16));
  if (role < 8) {
    const int g = wave & 3;    // group of a chunk
    const int rb = wave >> 2;  // 32-row block of the workgroup's 64 rows
    f32x16 acc[2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[cb][v] = 0.f;
      }
    }
    const uint32_t copy4 = static_cast<uint32_t>(lane & 31) << 2;
    const uint32_t x_lane = kXAddr + static_cast<uint32_t>(r * XS + 32 * h + 64 * g) * 2;
    const uint32_t w_lane =
        kWAddr + static_cast<uint32_t>((32 * rb + r) * kWideWStride + 32 * g + 16 * h);
    const uint32_t s_lane =
        kScaleAddr +
        static_cast<uint32_t>(g * ROWS + 32 * rb + 8 * ((lane & 15) >> 2) + 4 * h + (lane & 3)) * 2;
    for (int c = 0; c < n_ch; ++c) {
      const uint32_t buf = static_cast<uint32_t>(c & 1);
      const int grp = min(4 * c + g, groups - 1) - g;
      float mine = f16_to_f32(*reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(
          s_lane + static_cast<uint32_t>(grp * ROWS * 2)));
      const uint4 wv = lds0_u128(w_lane + buf * kWideWBytes);
      const uint32_t w4[4] = {wv.x, wv.y, wv.z, wv.w};
      const uint32_t xl = x_lane + buf * kWideXBytes;
      f32x16 t[2];
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          t[cb][v] = 0.f;
        }
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const uint32_t w = w4[jj];
        const uint4 a = make_uint4(pair32_at<0>(w, copy4), pair32_at<1>(w, copy4), pair32_at<2>(w, copy4),
                                   pair32_at<3>(w, copy4));
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
          const uint4 b = lds0_u128(xl + static_cast<uint32_t>(cb * 32 * XS * 2) + 16 * jj);
          t[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                          __builtin_bit_cast(bf16x8, b), t[cb], 0, 0, 0);
        }
      }
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        scale_into_all(acc[cb], mine, t[cb]);
      }
      __syncthreads();
    }
    // the four sums of every output (one per group of a chunk) meet in LDS
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        sums[((cb * 8 + wave) * 16 + v) * kWave + lane] = acc[cb][v];
      }
    }
  }
  __syncthreads();
  // wavefront w of the sixteen finishes accumulator value w of both row blocks and both
  // halves of the tokens
  float o32[4];
  size_t at[4];
  bool live[4];
  int orow[4];
#pragma unroll
  for (int o = 0; o < 4; ++o) {
    const int rb = o >> 1, cb = o & 1, v = wave16;
    o32[o] = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      o32[o] += sums[((cb * 8 + 4 * rb + g) * 16 + v) * kWave + lane];
    }
    const int rr = row_base + (PAIR ? 0 : 32 * rb) + 8 * (v >> 2) + 4 * h + (v & 3);
    live[o] = rr < M;
    orow[o] = out0 + min(rr, M - 1);
    // (row 32 cb + r of the chunk buffers holds token 4 (r % 16) + 2 cb + r / 16)
    at[o] = static_cast<size_t>(orow[o]) * N + 4 * (r & 15) + 2 * cb + (r >> 4);
  }
  if constexpr (PAIR) {
    // outputs 0, 1 are the gate's two token halves, 2, 3 the up's, at the same rows
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      if (live[cb]) {
        const float a = bf16_to_f32(f32_to_bf16(o32[cb]));
        const float act = bf16_to_f32(f32_to_bf16(a / (1.f + expf(-a))));
        y[at[cb]] = f32_to_bf16(act * bf16_to_f32(f32_to_bf16(o32[2 + cb])));
      }
    }
    return;
  }
  if (partial != nullptr) {
    const size_t slab = static_cast<size_t>(M_all) * N;
    if (arrive_slot < 0) {
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        if (live[o]) {
          partial[blockIdx.y * slab + at[o]] = o32[o];
        }
      }
      return;  // a reduce kernel adds the slabs up
    }
    // the splits meet here: see gemm_stream
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      if (live[o]) {
        __hip_atomic_store(partial + blockIdx.y * slab + at[o], o32[o], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int *last = reinterpret_cast<int *>(lds_raw + kScaleAddr);  // (the scales are done with)
    if (tid == 0) {
      unsigned int *count = &stream_arrivals[arrive_slot][blockIdx.x];
      const unsigned int before =
          __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool all_in = before + 1 == n_splits;
      if (all_in) {
        __hip_atomic_store(count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      *last = all_in ? 1 : 0;
    }
    __syncthreads();
    if (*last == 0) {
      return;
    }
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      float sum = 0.f;
      for (unsigned int j0 = 0; j0 < n_splits; j0 += 4) {
        float v[4];
#pragma unroll
        for (unsigned int u = 0; u < 4; ++u) {
          v[u] = __hip_atomic_load(partial + min(j0 + u, n_splits - 1) * slab + at[o], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (unsigned int u = 0; u < 4; ++u) {
          sum = j0 + u == 0 ? v[0] : (j0 + u < n_splits ? sum + v[u] : sum);
        }
      }
      o32[o] = sum;
    }
  }
  float square[4];
#pragma unroll
  for (int o = 0; o < 4; ++o) {
    square[o] = 0.f;
    if (live[o]) {
      uint16_t out = f32_to_bf16(o32[o]);
      if (bias != nullptr) {
        out = f32_to_bf16(bf16_to_f32(out) + bf16_to_f32(bias[orow[o]]));
      }
      if (res != nullptr) {
        out = f32_to_bf16(bf16_to_f32(res[at[o]]) + bf16_to_f32(out));
      }
      y[at[o]] = out;
      square[o] = bf16_to_f32(out) * bf16_to_f32(out);
    }
  }
  // The column sums of squares of what was stored, per block of 1024 / 64 = 16 rows (see
  // gemm_stream): rows 16 b .. + 16 of the workgroup's 64 are accumulator values 8 (b % 2) ..
  // + 8 of row block b / 2, in both halves of the lanes.
  if (colsq != nullptr) {
    __syncthreads();  // every wavefront is past its reads of `sums`
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      sums[(o * 16 + wave16) * kWave + lane] = square[o];
    }
    __syncthreads();
    if (tid < 256) {
      const int b = tid >> 6, col = tid & 63;
      const int cb = (col >> 1) & 1;
      const int rcol = (col >> 2) + 16 * (col & 1);  // the B operand's column of block cb that holds token col
      const int o = 2 * (b >> 1) + cb;
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        sum += sums[(o * 16 + 8 * (b & 1) + v) * kWave + rcol];
        sum += sums[(o * 16 + 8 * (b & 1) + v) * kWave + rcol + 32];
      }
      if (row_base + 16 * b < M) {
        colsq[static_cast<size_t>((row_base >> 4) + b) * 64 + col] = sum;
      }
    }
  }
}

struct RowsArgs {
  GemmSegs segs;
  const uint16_t *x;
  uint16_t *y;
  float *partial;
  int M_all, K, K_pad, N;
  const uint16_t *bias, *res;
};

template <bool VEC, int NC, int TPS>
int rows_one(const RowsArgs &a, dim3 grid, hipStream_t st, bool attr_only) {
  if (attr_only) {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_rows<VEC, NC, TPS>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               rows_lds_bytes(NC, TPS)) == hipSuccess
               ? 0
               : -6;
  }
  gemm_rows<VEC, NC, TPS><<<grid, dim3(kRowsBlock), rows_lds_bytes(NC, TPS), st>>>(
      a.segs, a.x, a.y, a.partial, a.M_all, a.K, a.K_pad, a.N, a.bias, a.res);
  return 0;
}

template <bool VEC, int NC>
int rows_by_tiles(int tps, const RowsArgs &a, dim3 grid, hipStream_t st, bool attr_only) {
  switch (tps) {
    case 1:
      return rows_one<VEC, NC, 1>(a, grid, st, attr_only);
    case 2:
      return rows_one<VEC, NC, 2>(a, grid, st, attr_only);
    case 3:
      if constexpr (NC < 4) return rows_one<VEC, NC, 3>(a, grid, st, attr_only);
      return -6;
    case 4:
      if constexpr (NC < 4) return rows_one<VEC, NC, 4>(a, grid, st, attr_only);
      return -6;
    default:
      return -6;
  }
}

// nc: 16-column blocks (1, 2 or 4).  attr_only raises the kernel's LDS limit instead of
// launching it.
int rows_dispatch(bool vec, int nc, int tps, const RowsArgs &a, dim3 grid, hipStream_t st,
                  bool attr_only) {
  if (vec) {
    return nc == 1   ? rows_by_tiles<true, 1>(tps, a, grid, st, attr_only)
           : nc == 2 ? rows_by_tiles<true, 2>(tps, a, grid, st, attr_only)
                     : rows_by_tiles<true, 4>(tps, a, grid, st, attr_only);
  }
  return nc == 1   ? rows_by_tiles<false, 1>(tps, a, grid, st, attr_only)
         : nc == 2 ? rows_by_tiles<false, 2>(tps, a, grid, st, attr_only)
                   : rows_by_tiles<false, 4>(tps, a, grid, st, attr_only);
}


// Sums of P elements over the splits, each in split order.  The loads of a batch of B splits
// are issued before the first add: written as a plain loop a sum is a chain of dependent trips
// to memory (load, wait, add), seven of them for a 5120-wide K.  Every load of a batch is
// unconditional -- a load under a branch is waited for where the branch ends -- and slots
// past the last split read split 0 again, their values unused; B is picked so that at most
// half the slots are such repeats (the partials are read with the streaming hint, a repeat
// is a second trip).  The first batch stands outside the loop, whose head waits for every
// load issued before it.
template <int P, int B>
__device__ __forceinline__ void sum_splits_by(const float *const (&p)[P], size_t stride,
                                              int split, float (&s)[P]) {
  float v[P][B];
#pragma unroll
  for (int u = 0; u < B; ++u) {
#pragma unroll
    for (int e = 0; e < P; ++e) {
      v[e][u] = __builtin_nontemporal_load(p[e] + (u < split ? u : 0) * stride);
    }
  }
#pragma unroll
  for (int e = 0; e < P; ++e) {
    s[e] = 0.f;
#pragma unroll
    for (int u = 0; u < B; ++u) {
      if (u < split) {
        s[e] += v[e][u];
      }
    }
  }
  for (int j0 = B; j0 < split; j0 += B) {
#pragma unroll
    for (int u = 0; u < B; ++u) {
#pragma unroll
      for (int e = 0; e < P; ++e) {
        v[e][u] = __builtin_nontemporal_load(p[e] + (j0 + u < split ? j0 + u : 0) * stride);
      }
    }
#pragma unroll
    for (int e = 0; e < P; ++e) {
#pragma unroll
      for (int u = 0; u < B; ++u) {
        if (j0 + u < split) {
          s[e] += v[e][u];
        }
      }
    }
  }
}

template <int P>
__device__ __forceinline__ void sum_splits(const float *const (&p)[P], size_t stride, int split,
                                           float (&s)[P]) {
  if (split <= 2) {
    sum_splits_by<P, 2>(p, stride, split, s);
  } else if (split <= 4) {
    sum_splits_by<P, 4>(p, stride, split, s);
  } else {
    sum_splits_by<P, 8>(p, stride, split, s);
  }
}

__device__ __forceinline__ float sum_splits(const float *p, size_t stride, int split) {
  const float *const ps[1] = {p};
  float s[1];
  sum_splits<1>(ps, stride, split, s);
  return s[0];
}

// y[i] = bf16( sum over splits, in split order, of partial[s][i] ), then optionally
// bf16(y + bias[row]) and bf16(res[i] + y): the roundings of separate bias and residual adds.
__global__ __launch_bounds__(256) void reduce_splitk(const float *__restrict__ partial,
                                                     uint16_t *__restrict__ y, int rows,
                                                     int split, int N,
                                                     const uint16_t *__restrict__ bias,
                                                     const uint16_t *res) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= rows) {
    return;
  }
  // Bias and residual are requested before the partials are waited for.  The loads are
  // unconditional (an absent operand reads y instead, a valid address whose value is not
  // used): a load under a branch is waited for where the branch ends.
  const uint16_t b = (bias != nullptr ? bias : y)[i / N];
  const uint16_t r = (res != nullptr ? res : y)[i];
  const float s = sum_splits(partial + i, static_cast<size_t>(rows), split);
  uint16_t v = f32_to_bf16(s);
  if (bias != nullptr) {
    v = f32_to_bf16(bf16_to_f32(v) + bf16_to_f32(b));
  }
  if (res != nullptr) {
    v = f32_to_bf16(bf16_to_f32(r) + bf16_to_f32(v));
  }
  y[i] = v;
}

// reduce_splitk that also leaves, for the RMSNorm that reads y next, the column sums of
// squares of what it stored: sq[b][n] = sum over the rows of block b of y[row][n]^2, taken
// from the bf16 values as stored.  A block is 1024 elements (1024 / N rows), one per thread as
// in reduce_splitk (fewer threads with more elements each were three times slower: the sums
// over the splits are chains of dependent loads).  N divides 256, so the threads of a column
// sit N apart; they are added in thread order (deterministic).
constexpr int kSqElems = 1024;  // elements of y per block of the sums = threads of a block

__global__ __launch_bounds__(kSqElems) void reduce_splitk_sq(const float *__restrict__ partial,
                                                             uint16_t *__restrict__ y, int rows,
                                                             int split, int N,
                                                             const uint16_t *__restrict__ bias,
                                                             const uint16_t *res,
                                                             float *__restrict__ sq) {
  __shared__ float part[kSqElems];
  const int i = blockIdx.x * kSqElems + threadIdx.x;
  float sqv = 0.f;
  if (i < rows) {
    const uint16_t b = (bias != nullptr ? bias : y)[i / N];  // unconditional, as in reduce_splitk
    const uint16_t r = (res != nullptr ? res : y)[i];
    const float s = sum_splits(partial + i, static_cast<size_t>(rows), split);
    uint16_t v = f32_to_bf16(s);
    if (bias != nullptr) {
      v = f32_to_bf16(bf16_to_f32(v) + bf16_to_f32(b));
    }
    if (res != nullptr) {
      v = f32_to_bf16(bf16_to_f32(r) + bf16_to_f32(v));
    }
    y[i] = v;
    const float f = bf16_to_f32(v);
    sqv = f * f;
  }
  part[threadIdx.x] = sqv;
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < N) {
    float t = 0.f;
    for (int k = threadIdx.x; k < kSqElems; k += N) {
      t += part[k];
    }
    sq[static_cast<size_t>(blockIdx.x) * N + threadIdx.x] = t;
  }
}

// Gate rows stacked over up rows: y[i] = silu(bf16 gate) * bf16 up with the roundings of the
// reference's separate ops (F.silu on bf16, then a bf16 product; gpu/decodev2/ops.py:23-24).
__global__ __launch_bounds__(256) void reduce_swiglu(const float *__restrict__ partial,
                                                     uint16_t *__restrict__ y, int half_rows,
                                                     int split) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= half_rows) {
    return;
  }
  const size_t stride = static_cast<size_t>(2) * half_rows;
  const float *const ps[2] = {partial + i, partial + half_rows + i};
  float gu[2];
  sum_splits<2>(ps, stride, split, gu);
  const float g = gu[0], u = gu[1];
  const float a = bf16_to_f32(f32_to_bf16(g));
  const float act = bf16_to_f32(f32_to_bf16(a / (1.f + expf(-a))));
  y[i] = f32_to_bf16(act * bf16_to_f32(f32_to_bf16(u)));
}

// The kernels use more than the default 64 KB of LDS: raise the limit once per process
// (on the first launch, which a caller warming up before graph capture makes eagerly).
int gemm_lds_ready() {
  static const int rc = [] {
    const std::pair<const void *, int> kernels[4] = {
        {reinterpret_cast<const void *>(gemm_mfma<true, 1>), gemm_lds_bytes(1)},
        {reinterpret_cast<const void *>(gemm_mfma<false, 1>), gemm_lds_bytes(1)},
        {reinterpret_cast<const void *>(gemm_mfma<true, 2>), gemm_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_mfma<false, 2>), gemm_lds_bytes(2)}};
    for (const auto &k : kernels) {
      if (hipFuncSetAttribute(k.first, hipFuncAttributeMaxDynamicSharedMemorySize, k.second) !=
          hipSuccess) {
        (void)hipGetLastError();
        return -6;
      }
    }
    const std::pair<const void *, int> streams[11] = {
        {reinterpret_cast<const void *>(gemm_stream<1, 2, true>), stream_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_stream<2, 2, true>), stream_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_stream<4, 2, true>), stream_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_stream64<false>), kWideLdsBytes},
        {reinterpret_cast<const void *>(gemm_stream64<true>), kWideLdsBytes},
        {reinterpret_cast<const void *>(gemm_stream<1, 1>), stream_lds_bytes(1)},
        {reinterpret_cast<const void *>(gemm_stream<2, 1>), stream_lds_bytes(1)},
        {reinterpret_cast<const void *>(gemm_stream<4, 1>), stream_lds_bytes(1)},
        {reinterpret_cast<const void *>(gemm_stream<1, 2>), stream_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_stream<2, 2>), stream_lds_bytes(2)},
        {reinterpret_cast<const void *>(gemm_stream<4, 2>), stream_lds_bytes(2)}};
    for (const auto &k : streams) {
      if (hipFuncSetAttribute(k.first, hipFuncAttributeMaxDynamicSharedMemorySize, k.second) !=
          hipSuccess) {
        (void)hipGetLastError();
        return -6;
      }
    }
    const RowsArgs none{};
    for (int vec = 0; vec < 2; ++vec) {
      for (int nc = 1; nc <= 4; nc *= 2) {
        for (int tps = 1; tps <= rows_max_tiles(nc); ++tps) {
          if (rows_dispatch(vec != 0, nc, tps, none, dim3(1), nullptr, true) != 0) {
            (void)hipGetLastError();
            return -6;
          }
        }
      }
    }
    return 0;
  }();
  return rc;
}

}  // namespace
}  // namespace chr

using namespace chr;

extern "C" void chr_nf4_gemm_stream_policy(int32_t policy) {
  chr::stream_policy().store(policy < 0 ? -1 : (policy > 0 ? 1 : 0), std::memory_order_relaxed);
}

extern "C" void chr_nf4_set_tuning(int32_t path, int32_t split_k, int32_t one_wave) {
  Tuning &t = tuning();
  t.path = (path >= 0 && path <= 2) ? path : 0;
  t.split_k = split_k > 0 ? split_k : 0;
  t.one_wave = one_wave > 0 ? one_wave : 0;
}

extern "C" int chr_nf4_gemm_plan(const chr_nf4_dev_t *w, int32_t N, int32_t have_ws,
                                 chr_nf4_plan_t *out) {
  if (out == nullptr) {
    return -1;
  }
  chr_nf4_dev_t h{};
  const int rc = check_args(w, N, /*need_ptrs=*/false, &h, kPlanMaxN);
  if (rc != 0) {
    return rc;
  }
  return plan_impl(h, N, have_ws, out);
}

namespace chr {
namespace {

// Grid, split and workspace of a launch over nseg stacked matrices (nseg == 1: plan_impl).
struct StackPlan {
  GemmSegs segs;
  int M_all, grid_x, grid_y, n_ktiles, tiles_per_split;
  int64_t ws_floats;
  int stream;  // 32-row blocks of a workgroup of the stream tile, 0: another tile
};

// The row of arrival counts a split launch of the stream tile uses, or -1: its splits then meet
// in a reduce kernel, which needs no counts (and gives the same bits).  Two launches may share a
// row only if they cannot run at the same time:
//   - eager launches on one stream run one after the other: a row per (device, stream);
//   - a launch recorded during stream capture runs whenever and wherever its graph is replayed,
//     possibly beside eager work on the stream it was captured from: a row per (device,
//     capture, stream), which no eager launch and no other graph ever gets (two replays of one
//     graph do not overlap: the runtime orders launches of one executable graph);
//   - the per-thread default stream is one handle for many streams: no row, -1.
// Rows are never handed back (nothing tells the library that a graph is gone); when all 512
// are taken, further owners get -1.
int arrival_slot(hipStream_t st) {
  struct Owner {
    int dev;
    hipStream_t st;
    unsigned long long capture;  // 0: eager launches on st
  };
  static std::mutex mu;
  static Owner owner[kArriveSlots];
  static int used = 0;
  if (st == hipStreamPerThread) {
    return -1;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  unsigned long long capture = 0;
  {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if (hipStreamGetCaptureInfo(st, &status, &id) != hipSuccess) {
      (void)hipGetLastError();
      return -1;
    }
    if (status == hipStreamCaptureStatusActive) {
      capture = id + 1;  // (ids start anywhere: keep 0 for "not capturing")
    } else if (status != hipStreamCaptureStatusNone) {
      return -1;  // a capture that has been invalidated: the launch will fail anyway
    }
  }
  const std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i) {
    if (owner[i].dev == dev && owner[i].st == st && owner[i].capture == capture) {
      return i;
    }
  }
  if (used == kArriveSlots) {
    return -1;
  }
  owner[used] = {dev, st, capture};
  return used++;
}

// allow_stream: false when the launch cannot take the stream tile for a reason the shape does
// not show (scales not 8-byte aligned).
StackPlan plan_stack(const chr_nf4_dev_t *h, int nseg, int N, int have_ws, bool allow_stream = true) {
  StackPlan sp{};
  int blocks32 = 0, blocks64 = 0;
  for (int i = 0; i < nseg; ++i) {
    blocks32 += ceil_div(h[i].M, kStreamRows);
    blocks64 += ceil_div(h[i].M, 2 * kStreamRows);
  }
  int64_t codes = 0;
  for (int i = 0; i < nseg; ++i) {
    codes += static_cast<int64_t>(h[i].M) * h[i].K_pad;
  }
  const StreamPlan stp = allow_stream ? stream_plan(N, h[0].K_pad, blocks32, blocks64, have_ws, codes)
                                      : StreamPlan{0, 1, 0};
  sp.stream = stp.rb;
  const int bm = sp.stream ? kStreamRows * sp.stream : kBM;
  for (int i = 0; i < 3; ++i) {
    const bool on = i < nseg;
    sp.segs.packed[i] = on ? h[i].packed : nullptr;
    sp.segs.scale[i] = on ? h[i].scale : nullptr;
    sp.segs.M[i] = on ? h[i].M : 0;
    sp.segs.blocks[i] = on ? ceil_div(h[i].M, bm) : 0;
    sp.segs.row0[i] = sp.M_all;
    sp.M_all += sp.segs.M[i];
    sp.grid_x += sp.segs.blocks[i];
  }
  sp.n_ktiles = ceil_div(h[0].K_pad, kBK);
  if (sp.stream) {
    sp.grid_y = stp.split;
    sp.tiles_per_split = N == 64 ? stp.chunks : std::min(2 * stp.chunks, sp.n_ktiles);
    sp.ws_floats = sp.grid_y > 1 ? static_cast<int64_t>(sp.grid_y) * sp.M_all * N : 0;
    return sp;
  }
  pick_split(sp.grid_x, sp.n_ktiles, N, have_ws, &sp.grid_y, &sp.tiles_per_split);
  sp.ws_floats = sp.grid_y > 1 ? static_cast<int64_t>(sp.grid_y) * sp.M_all * N : 0;
  return sp;
}

// Whether a stacked gate+up launch pairs the rows inside the tile (its unsplit 64-row forms):
// then there are no partials and no reduce launch.
bool swiglu_pairs(const StackPlan &sp, int /*N*/) { return sp.stream == 2 && sp.grid_y == 1; }

// live_max: widest chunk the entry launches.  The reference's entries stop at 32 columns
// (wider ones are described by the planner only); the chr_dv2_gemm_* entries go to 64.
// w[0..nseg) share K and x; y, bias and res cover the stacked rows.
int gemm_launch(const chr_nf4_dev_t *const *w, int nseg, const void *x, void *y, int32_t N,
                float *ws, int64_t ws_floats, void *stream, int32_t max_n, const void *bias,
                const void *res, int32_t live_max = kLiveMaxN, bool swiglu = false,
                float *colsq = nullptr) {
  if (x == nullptr || y == nullptr) {
    return -1;
  }
  if (max_n < 1 || max_n > kPlanMaxN) {
    return -2;
  }
  chr_nf4_dev_t h[3] = {};
  for (int i = 0; i < nseg; ++i) {
    const int rc = check_args(w[i], N, /*need_ptrs=*/true, &h[i], max_n);
    if (rc != 0) {
      return rc;
    }
    if (h[i].K != h[0].K || h[i].K_pad != h[0].K_pad) {
      return -3;  // stacked matrices multiply the same x
    }
  }
  if (N > live_max) {
    return -2;
  }
  for (int i = 0; i < nseg; ++i) {
    if (!aligned16(h[i].packed) || !aligned2(h[i].scale)) {
      return -5;
    }
  }
  if (!aligned16(x)) {
    return -5;
  }
  if (N == 1) {
    if (bias != nullptr || res != nullptr || nseg != 1) {
      return -2;  // the fused epilogue and the stacking belong to the tiles (N >= 2)
    }
    return gemv_entry(&h[0], x, y, stream, nullptr, nullptr, 0.f, nullptr, nullptr);
  }
  const int have_ws = (ws != nullptr && ws_floats > 0) ? 1 : 0;
  bool scales_aligned8 = true;
  for (int i = 0; i < nseg; ++i) {
    scales_aligned8 = scales_aligned8 && (reinterpret_cast<uintptr_t>(h[i].scale) & 7u) == 0;
  }
  StackPlan sp = plan_stack(h, nseg, N, have_ws, scales_aligned8);
  bool pair = false;
  if (swiglu) {
    if (nseg != 2 || h[0].M != h[1].M || bias != nullptr || res != nullptr) {
      return -3;
    }
    pair = swiglu_pairs(sp, N);
    if (pair) {
      // a workgroup takes 32 gate rows and the 32 up rows that go with them, and stores the
      // activation itself
      sp.grid_x = ceil_div(h[0].M, kStreamRows);
      sp.segs.blocks[0] = sp.grid_x;
      sp.segs.blocks[1] = 0;
      sp.ws_floats = 0;
    } else {
      // the activation lives in the reduce, so the launch goes through fp32 partials
      sp.ws_floats = static_cast<int64_t>(sp.grid_y) * sp.M_all * N;
    }
  }
  if (sp.ws_floats > 0 && (!have_ws || ws_floats < sp.ws_floats)) {
    return -7;
  }
  float *partial = (sp.grid_y > 1 || (swiglu && !pair)) ? ws : nullptr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(sp.grid_x), static_cast<unsigned>(sp.grid_y));
  if (sp.stream != 0) {
    // whole chunks of K per workgroup of a row block: chunks of 256 at 64 columns, of 512 below
    const int chunk_k = (sp.stream == 2 && N == 64) ? kWideChunkK : kStreamChunkK;
    sp.segs.splits = sp.grid_y;
    sp.segs.per_split = ceil_div(ceil_div(h[0].K_pad, chunk_k), sp.grid_y);
  }
  // 16-byte activation vectors need N in {8, 16, 32, 64}; x is 16-byte aligned (checked above)
  const bool vec = N == 8 || N == 16 || N == 32 || N == 64;
  if (gemm_lds_ready() != 0) {
    return -6;
  }
  const auto *xp = static_cast<const uint16_t *>(x);
  auto *yp = static_cast<uint16_t *>(y);
  const auto *bp = static_cast<const uint16_t *>(bias);
  const auto *rp = static_cast<const uint16_t *>(res);
  const dim3 block(kGemmBlock);
  const int K = h[0].K, K_pad = h[0].K_pad;
  const int nc = rows_col_blocks(N);
  // the stream tile's splits meet in the tile itself unless the reduce has more to do
  // (SwiGLU, the column sums of squares)
  // (at 32 and 64 columns the tile leaves the column sums of squares itself)
  const bool sq_in_tile = colsq != nullptr && nseg == 1 && sp.stream != 0 && (N == 32 || N == 64);
  float *tile_sq = sq_in_tile ? colsq : nullptr;
  int slot = -1;
  if (sp.stream != 0 && sp.grid_y > 1 && !swiglu && (sq_in_tile || !(colsq != nullptr && 256 % N == 0))) {
    slot = sp.grid_x <= kArriveBlocks ? arrival_slot(st) : -1;
  }
  if (sp.stream == 1) {
    if (N <= 16) {
      gemm_stream<1, 1><<<grid, dim3(kStreamBlock), stream_lds_bytes(1), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    } else if (N == 32) {
      gemm_stream<4, 1><<<grid, dim3(kStreamBlock), stream_lds_bytes(1), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    } else {
      gemm_stream<2, 1><<<grid, dim3(kStreamBlock), stream_lds_bytes(1), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    }
  } else if (sp.stream == 2 && N == 64) {
    if (pair) {
      gemm_stream64<true><<<grid, dim3(kStreamBlock), kWideLdsBytes, st>>>(sp.segs, xp, yp, nullptr, sp.M_all,
                                                                            K, K_pad, nullptr, nullptr, -1,
                                                                            nullptr);
      return launch_rc();
    }
    gemm_stream64<false><<<grid, dim3(kStreamBlock), kWideLdsBytes, st>>>(sp.segs, xp, yp, partial, sp.M_all,
                                                                           K, K_pad, bp, rp, slot, tile_sq);
  } else if (sp.stream == 2 && pair) {
    if (N <= 16) {
      gemm_stream<1, 2, true><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, nullptr, sp.M_all, K, K_pad, N, nullptr, nullptr, -1, nullptr);
    } else if (N == 32) {
      gemm_stream<4, 2, true><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, nullptr, sp.M_all, K, K_pad, N, nullptr, nullptr, -1, nullptr);
    } else {
      gemm_stream<2, 2, true><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, nullptr, sp.M_all, K, K_pad, N, nullptr, nullptr, -1, nullptr);
    }
    return launch_rc();
  } else if (sp.stream == 2) {
    if (N <= 16) {
      gemm_stream<1, 2><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    } else if (N == 32) {
      gemm_stream<4, 2><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    } else {
      gemm_stream<2, 2><<<grid, dim3(kStreamBlock), stream_lds_bytes(2), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp, slot, tile_sq);
    }
  } else if (rows_kernel_serves(N, sp.tiles_per_split)) {
    const RowsArgs ra{sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, bp, rp};
    // the vector staging needs whole 16-byte vectors per row of x
    if (rows_dispatch((N & 7) == 0, nc, sp.tiles_per_split, ra, grid, st, false) != 0) {
      return -6;
    }
  } else if (N <= kBN) {
    if (vec) {
      gemm_mfma<true, 1><<<grid, block, gemm_lds_bytes(1), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, sp.n_ktiles, sp.tiles_per_split, bp, rp);
    } else {
      gemm_mfma<false, 1><<<grid, block, gemm_lds_bytes(1), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, sp.n_ktiles, sp.tiles_per_split, bp, rp);
    }
  } else {
    if (vec) {
      gemm_mfma<true, 2><<<grid, block, gemm_lds_bytes(2), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, sp.n_ktiles, sp.tiles_per_split, bp, rp);
    } else {
      gemm_mfma<false, 2><<<grid, block, gemm_lds_bytes(2), st>>>(
          sp.segs, xp, yp, partial, sp.M_all, K, K_pad, N, sp.n_ktiles, sp.tiles_per_split, bp, rp);
    }
  }
  if (swiglu) {
    const int half_rows = h[0].M * N;
    reduce_swiglu<<<dim3(static_cast<unsigned>(ceil_div(half_rows, 256))), dim3(256), 0, st>>>(
        partial, yp, half_rows, sp.grid_y);
  } else if (partial != nullptr && slot < 0) {
    const int rows = sp.M_all * N;
    if (colsq != nullptr && 256 % N == 0) {
      reduce_splitk_sq<<<dim3(static_cast<unsigned>(ceil_div(rows, kSqElems))), dim3(kSqElems),
                         0, st>>>(partial, yp, rows, sp.grid_y, N, bp, rp, colsq);
      return launch_rc();
    }
    reduce_splitk<<<dim3(static_cast<unsigned>(ceil_div(rows, 256))), dim3(256), 0, st>>>(
        partial, yp, rows, sp.grid_y, N, bp, rp);
  }
  const int rc = launch_rc();
  if (sq_in_tile && (partial == nullptr || slot >= 0)) {
    return rc;  // the tile wrote them
  }
  // a caller that asked for the column sums learns that this launch did not write them
  return rc == 0 && colsq != nullptr ? 1 : rc;
}

}  // namespace
}  // namespace chr

extern "C" int chr_nf4_gemm_ws_max(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                                   float *ws, int64_t ws_floats, void *stream, int32_t max_n) {
  return gemm_launch(&w, 1, x, y, N, ws, ws_floats, stream, max_n, nullptr, nullptr);
}

extern "C" int chr_dv2_gemm_add(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                                float *ws, int64_t ws_floats, const void *bias,
                                const void *residual, void *stream) {
  return gemm_launch(&w, 1, x, y, N, ws, ws_floats, stream, kPlanMaxN, bias, residual, kPlanMaxN);
}

extern "C" int chr_dv2_gemm_add_sq(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                                   float *ws, int64_t ws_floats, const void *bias,
                                   const void *residual, float *colsq, void *stream) {
  if (colsq == nullptr) {
    return -1;
  }
  return gemm_launch(&w, 1, x, y, N, ws, ws_floats, stream, kPlanMaxN, bias, residual, kPlanMaxN,
                     false, colsq);
}

extern "C" int32_t chr_dv2_sq_rows(int32_t N) {
  return N >= 1 && N <= kSqElems && kSqElems % N == 0 ? kSqElems / N : 0;
}

extern "C" int64_t chr_dv2_gemm_qkv_ws(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                                       const chr_nf4_dev_t *v, int32_t N) {
  if (q == nullptr || k == nullptr || v == nullptr || N < 2 || N > kPlanMaxN) {
    return -1;
  }
  const chr_nf4_dev_t h[3] = {*q, *k, *v};
  if (h[0].M < 1 || h[1].M < 1 || h[2].M < 1 || h[0].K < 1 || !k_pad_ok(h[0].K, h[0].K_pad)) {
    return -1;
  }
  return plan_stack(h, 3, N, 1).ws_floats;
}

extern "C" int chr_dv2_gemm_qkv(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                                const chr_nf4_dev_t *v, const void *x, void *y, int32_t N,
                                float *ws, int64_t ws_floats, const void *bias, void *stream) {
  if (q == nullptr || k == nullptr || v == nullptr) {
    return -1;
  }
  const chr_nf4_dev_t *w[3] = {q, k, v};
  return gemm_launch(w, 3, x, y, N, ws, ws_floats, stream, kPlanMaxN, bias, nullptr, kPlanMaxN);
}

extern "C" int chr_nf4_gemm_ws(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                               float *ws, int64_t ws_floats, void *stream) {
  return chr_nf4_gemm_ws_max(w, x, y, N, ws, ws_floats, stream, kLiveMaxN);
}

extern "C" int chr_nf4_gemm(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                            void *stream) {
  return chr_nf4_gemm_ws(w, x, y, N, nullptr, 0, stream);
}

// ---- a GEMM entry that allocates nothing ----------------------------------------------------
// The split-K partials of chr_nf4_gemm_ws live in a workspace the caller allocates.  This
// entry keeps them in a file-scope device array instead, for callers that cannot allocate
// (code under graph capture, tight serving loops).  Every device the library runs on holds
// its own copy of the array, at its own address, until the process ends.
namespace {

constexpr int64_t kScratchFloats = int64_t{4} << 20;  // 16 MiB of fp32 partials
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;

// Device address of this device's copy of the array; null if the runtime refuses.  The
// array's name is only a handle in host code: the address a kernel can use comes from
// hipGetSymbolAddress, once per device, with that device current.
float *scratch_on_current_device() {
  static std::atomic<float *> known[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  float *p = known[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void *addr = nullptr;
    if (hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)) != hipSuccess || addr == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    p = static_cast<float *>(addr);
    known[dev].store(p, std::memory_order_release);  // racing first calls store the same value
  }
  return p;
}

}  // namespace

extern "C" int64_t chr_nf4_gemm_noalloc_max_floats(void) { return kScratchFloats; }

extern "C" int chr_nf4_gemm_noalloc(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                                    void *stream) {
  float *ws = scratch_on_current_device();
  if (ws == nullptr) {
    return -6;
  }
  // Same planner, same kernels and the same order of sums as chr_nf4_gemm_ws with a workspace
  // of kScratchFloats floats: a launch whose partials do not fit comes back as -7 from the
  // size check below, before anything is launched.  The partials need no clearing: every
  // split writes its whole [M, N] slab before the reduce reads it.
  return chr_nf4_gemm_ws(w, x, y, N, ws, kScratchFloats, stream);
}

extern "C" int64_t chr_dv2_gemm_swiglu_ws(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                                          int32_t N) {
  if (gate == nullptr || up == nullptr || N < 2 || N > kPlanMaxN) {
    return -1;
  }
  const chr_nf4_dev_t h[2] = {*gate, *up};
  if (h[0].M < 1 || h[0].M != h[1].M || h[0].K < 1 || !k_pad_ok(h[0].K, h[0].K_pad)) {
    return -1;
  }
  // (as the launch decides: the tile wants the scale blobs 8-byte aligned)
  const bool aligned = ((reinterpret_cast<uintptr_t>(h[0].scale) | reinterpret_cast<uintptr_t>(h[1].scale)) & 7u) == 0;
  const StackPlan sp = plan_stack(h, 2, N, 1, aligned);
  return swiglu_pairs(sp, N) ? 0 : static_cast<int64_t>(sp.grid_y) * sp.M_all * N;
}

extern "C" int chr_dv2_gemm_swiglu(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                                   const void *x, void *y, int32_t N, float *ws,
                                   int64_t ws_floats, void *stream) {
  if (gate == nullptr || up == nullptr) {
    return -1;
  }
  const chr_nf4_dev_t *w[2] = {gate, up};
  return gemm_launch(w, 2, x, y, N, ws, ws_floats, stream, kPlanMaxN, nullptr, nullptr, kPlanMaxN,
                     /*swiglu=*/true);
}

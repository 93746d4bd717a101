// Chunked-prefill NF4 GEMM for gfx950: y[M,N] = dequant(W[M,K]) @ x[K,N],
// N <= 32 token columns, on the CDNA4 bf16 matrix cores.  Also the launch
// planner, the split-K reduction and the chr_nf4_gemm* entry points.
// Replaces gpu/nf4/nf4_gemm.cu:665-678 (reduce), 933-1450 (prefill tiles),
// 1497-1785 (tuning, planner, entry points).
//
// Tile.  A workgroup is four wavefronts and owns 128 output rows; each
// wavefront owns 32 of them and all N columns, accumulating one 32x32 fp32
// tile with v_mfma_f32_32x32x16_bf16.  For that instruction lane l supplies
// A[row l%32][k 8*(l/32) .. +8) and B[k 8*(l/32) .. +8)][col l%32], eight
// consecutive k each, i.e. exactly one packed dword of codes on the A side.
// A lane therefore loads 16 bytes (32 codes) of its own row per 64-wide K
// step, rebuilds bf16(LUT*scale) pairs in registers and feeds four MFMAs;
// lanes l and l+32 read adjacent 16-byte pieces of the same row.
//
// The activation tile [BK=256, N] is staged once per workgroup in LDS,
// transposed to [32][BK+8] bf16 (token-major, padded so the 16-byte B reads of
// 32 lanes fall in distinct banks), and shared by the four wavefronts.
// Columns >= N and rows >= K are zero-filled, so padding codes and the unused
// MFMA columns contribute nothing.
//
// Split-K over grid.y writes fp32 partials [split][M][N] to the caller's
// workspace; a second kernel adds them in split order (deterministic) and
// rounds once to bf16.
//
// Numerics (gpu/nf4/nf4_gemm.cu:168-172, 312-323): weight = bf16(LUT*scale),
// bf16 x bf16 products, fp32 accumulate, one bf16 rounding of y.

#include "nf4_common.h"

#include <algorithm>
#include <cstdlib>

namespace chr {

int gemv_entry(const chr_nf4_dev_t *w, const void *x, void *y, void *stream, const void *add,
               const void *rms_w, float rms_eps);
int gemv_rows_per_wg(int M, int K_pad);
int gemv_threads_per_wg(int M, int K_pad);
int gemv_lds_bytes(int K_pad);

namespace {

constexpr int kLiveMaxN = 32;
constexpr int kPlanMaxN = 64;

constexpr int kBM = 128;      // rows per workgroup
constexpr int kBK = 256;      // K per staged activation tile
constexpr int kBN = 32;       // token columns of the MFMA tile
constexpr int kGemmBlock = 256;
constexpr int kXPad = 8;      // bf16 elements of row padding in LDS
constexpr int kXStride = kBK + kXPad;
constexpr int kGemmLds = kBN * kXStride * 2;

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

// split so that grid_x * split reaches two workgroups per compute unit, capped
// at the number of K tiles; split is recomputed from tiles_per_split so the
// pair always agrees with what the kernel indexes
// (gpu/nf4/nf4_gemm.cu:1526-1543).
void pick_split(int grid_x, int n_ktiles, int have_ws, int *split, int *tiles_per_split) {
  const Tuning &t = tuning();
  int want = 1;
  if (have_ws) {
    const int target = resolved_one_wave() * 2;
    want = t.split_k > 0 ? t.split_k : ceil_div(target, grid_x);
  }
  want = std::max(1, std::min(want, n_ktiles));
  const int tps = ceil_div(n_ktiles, want);
  *tiles_per_split = tps;
  *split = ceil_div(n_ktiles, tps);
}

int plan_impl(const chr_nf4_dev_t &h, int32_t N, int32_t have_ws, chr_nf4_plan_t *out) {
  chr_nf4_plan_t p{};
  if (N == 1) {
    // Row-streaming GEMV: every wavefront walks whole rows, no split-K.
    p.path = 1;
    p.bm = gemv_rows_per_wg(h.M, h.K_pad);
    p.bk = 2048;  // codes one wavefront load step covers
    p.block = gemv_threads_per_wg(h.M, h.K_pad);
    p.grid_x = ceil_div(h.M, p.bm);
    p.grid_y = 1;
    p.n_ktiles = ceil_div(h.K_pad, p.bk);
    p.tiles_per_split = p.n_ktiles;
    p.smem_bytes = gemv_lds_bytes(h.K_pad);
    p.ws_floats = 0;
  } else {
    p.path = N <= 16 ? 2 : (N <= 32 ? 3 : 4);
    p.bm = kBM;
    p.bk = kBK;
    p.block = kGemmBlock;
    p.grid_x = ceil_div(h.M, kBM);
    p.n_ktiles = ceil_div(h.K_pad, kBK);
    pick_split(p.grid_x, p.n_ktiles, have_ws, &p.grid_y, &p.tiles_per_split);
    p.smem_bytes = (N <= 32 ? 1 : 2) * kGemmLds;
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

// Stage x[k0 .. k0+kBK) x [0, N) into LDS as xs[n][k - k0] (bf16), zero where
// k >= K or n >= N.  x is [K, N] row-major.
__device__ __forceinline__ void stage_x(const uint16_t *__restrict__ x, uint16_t *xs, int k0,
                                        int K, int N) {
  // 256 threads walk (k, n) with n fastest: consecutive threads read
  // consecutive global elements.
  for (int i = threadIdx.x; i < kBK * kBN; i += kGemmBlock) {
    const int kk = i / kBN;
    const int n = i - kk * kBN;
    const int k = k0 + kk;
    uint16_t v = 0;
    if (n < N && k < K) {
      v = x[static_cast<size_t>(k) * N + n];
    }
    xs[n * kXStride + kk] = v;
  }
}

// Vector variant for N == 32 with a 16-byte aligned x: one thread moves eight
// consecutive tokens of one k.
__device__ __forceinline__ void stage_x_n32(const uint16_t *__restrict__ x, uint16_t *xs, int k0,
                                            int K) {
  for (int i = threadIdx.x; i < kBK * 4; i += kGemmBlock) {
    const int kk = i >> 2;
    const int n0 = (i & 3) * 8;
    const int k = k0 + kk;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (k < K) {
      v = *reinterpret_cast<const uint4 *>(x + static_cast<size_t>(k) * 32 + n0);
    }
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      xs[(n0 + 2 * j) * kXStride + kk] = static_cast<uint16_t>(w[j] & 0xFFFFu);
      xs[(n0 + 2 * j + 1) * kXStride + kk] = static_cast<uint16_t>(w[j] >> 16);
    }
  }
}

__device__ __forceinline__ bf16x8 dequant8(uint32_t w, float s, const float *lut) {
  bf16x8 a;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = static_cast<__bf16>(lut[(w >> (4 * j)) & 0xFu] * s);
  }
  return a;
}

__global__ __launch_bounds__(kGemmBlock) void gemm_mfma(const uint8_t *__restrict__ packed,
                                                        const uint16_t *__restrict__ scale,
                                                        const uint16_t *__restrict__ x,
                                                        uint16_t *__restrict__ y,
                                                        float *__restrict__ partial, int M, int K,
                                                        int K_pad, int N, int n_ktiles,
                                                        int tiles_per_split, int x_vec) {
  __shared__ float lut[16];
  __shared__ __attribute__((aligned(16))) uint16_t xs[kBN * kXStride];
  if (threadIdx.x < 16) {
    lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int row = blockIdx.x * kBM + wave * 32 + (lane & 31);
  const int rowc = min(row, M - 1);  // clamp: rows past M compute but never store
  const int khalf = lane >> 5;       // which 32-wide half of a 64-wide K step
  const uint8_t *prow = packed + static_cast<size_t>(rowc) * (K_pad >> 1);
  const uint16_t *srow = scale + static_cast<size_t>(rowc) * (K_pad >> 6);

  const int tile0 = blockIdx.y * tiles_per_split;
  const int tile1 = min(tile0 + tiles_per_split, n_ktiles);

  f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint16_t *xl = xs + (lane & 31) * kXStride + khalf * 32;

  for (int tile = tile0; tile < tile1; ++tile) {
    const int k0 = tile * kBK;
    __syncthreads();  // previous tile's readers are done (and the LUT is visible)
    if (x_vec) {
      stage_x_n32(x, xs, k0, K);
    } else {
      stage_x(x, xs, k0, K, N);
    }
    __syncthreads();
    const int kend = min(kBK, K_pad - k0);
    for (int kk = 0; kk < kend; kk += 64) {
      const int k = k0 + kk + khalf * 32;
      const uint4 pk = *reinterpret_cast<const uint4 *>(prow + (k >> 1));
      const float s = f16_to_f32(srow[k >> 6]);
      const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bf16x8 a = dequant8(w[t], s, lut);
        const bf16x8 b = *reinterpret_cast<const bf16x8 *>(xl + kk + 8 * t);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
      }
    }
  }

  // acc[i] is C[row 8*(i/4) + 4*(lane/32) + i%4][col lane%32] of the 32x32 tile.
  const int n = lane & 31;
  const int rbase = blockIdx.x * kBM + wave * 32 + 4 * (lane >> 5);
  if (n < N) {
    if (partial == nullptr) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = rbase + 8 * (i >> 2) + (i & 3);
        if (r < M) {
          y[static_cast<size_t>(r) * N + n] = f32_to_bf16(acc[i]);
        }
      }
    } else {
      float *p = partial + static_cast<size_t>(blockIdx.y) * M * N;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int r = rbase + 8 * (i >> 2) + (i & 3);
        if (r < M) {
          p[static_cast<size_t>(r) * N + n] = acc[i];
        }
      }
    }
  }
}

// y[i] = bf16( sum over splits, in split order, of partial[s][i] ).
__global__ __launch_bounds__(256) void reduce_splitk(const float *__restrict__ partial,
                                                     uint16_t *__restrict__ y, int rows,
                                                     int split) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= rows) {
    return;
  }
  float s = 0.f;
  for (int j = 0; j < split; ++j) {
    s += partial[static_cast<size_t>(j) * rows + i];
  }
  y[i] = f32_to_bf16(s);
}

}  // namespace
}  // namespace chr

using namespace chr;

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

extern "C" int chr_nf4_gemm_ws_max(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                                   float *ws, int64_t ws_floats, void *stream, int32_t max_n) {
  if (x == nullptr || y == nullptr) {
    return -1;
  }
  if (max_n < 1 || max_n > kPlanMaxN) {
    return -2;
  }
  chr_nf4_dev_t h{};
  const int rc = check_args(w, N, /*need_ptrs=*/true, &h, max_n);
  if (rc != 0) {
    return rc;
  }
  if (N > kLiveMaxN) {
    return -2;  // no 64-column tile is built
  }
  if (!aligned16(h.packed) || !aligned16(x) || !aligned2(h.scale)) {
    return -5;
  }
  if (N == 1) {
    return gemv_entry(&h, x, y, stream, nullptr, nullptr, 0.f);
  }
  const int have_ws = (ws != nullptr && ws_floats > 0) ? 1 : 0;
  chr_nf4_plan_t p{};
  plan_impl(h, N, have_ws, &p);
  if (p.ws_floats > 0 && (!have_ws || ws_floats < p.ws_floats)) {
    return -7;
  }
  float *partial = p.grid_y > 1 ? ws : nullptr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(p.grid_x), static_cast<unsigned>(p.grid_y));
  const int x_vec = (N == 32) ? 1 : 0;
  gemm_mfma<<<grid, dim3(kGemmBlock), 0, st>>>(h.packed, h.scale,
                                               static_cast<const uint16_t *>(x),
                                               static_cast<uint16_t *>(y), partial, h.M, h.K,
                                               h.K_pad, N, p.n_ktiles, p.tiles_per_split, x_vec);
  if (partial != nullptr) {
    const int rows = h.M * N;
    reduce_splitk<<<dim3(static_cast<unsigned>(ceil_div(rows, 256))), dim3(256), 0, st>>>(
        partial, static_cast<uint16_t *>(y), rows, p.grid_y);
  }
  return launch_rc();
}

extern "C" int chr_nf4_gemm_ws(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                               float *ws, int64_t ws_floats, void *stream) {
  return chr_nf4_gemm_ws_max(w, x, y, N, ws, ws_floats, stream, kLiveMaxN);
}

extern "C" int chr_nf4_gemm(const chr_nf4_dev_t *w, const void *x, void *y, int32_t N,
                            void *stream) {
  return chr_nf4_gemm_ws(w, x, y, N, nullptr, 0, stream);
}

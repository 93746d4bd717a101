// Glue kernels of the chunked prefill for gfx950 (MI355X), all on the layout the prefill GEMM
// reads and writes: feature-major [features, N] bf16 with the N tokens of the chunk fastest
// (N <= 64, the widest chunk chr_dv2_gemm_add multiplies).  With them a prefill layer needs no
// transposes between its GEMMs.  They stand in for the stock torch ops of the reference's prefill (gpu/decodev2/prefill.py:58-133,
// gpu/decodev2/ops.py:18-44): RMSNorm, rotate-half RoPE + cache write, SwiGLU, bias/residual.

#include "nf4_common.h"

namespace chr {
namespace {

constexpr int kColsBlock = 1024;
constexpr int kColsWaves = kColsBlock / kWave;
constexpr int kMaxCols = 64;

// y[k][n] = bf16( (w[k] * x[k][n]) * rsqrt(mean_k x[k][n]^2 + eps) ).  Every workgroup needs the
// column sums of squares of the whole tile and then normalises its own slice of rows: one
// launch, no cross-workgroup hand-over.  The sums come from one of two places:
//   sq == nullptr: the workgroup reads the whole tile itself (a few hundred KB, in L2; all
//                  workgroups add in one order, so all hold the same bits);
//   sq != nullptr: the launch that stored x left sums per block of rows, sq[sq_blocks][N]
//                  (chr_dv2_gemm_add_sq), and only those are added.  N divides 1024 then.
//
// Thread t owns column t % CP of rows t / CP, t / CP + 1024 / CP, ..; CP is N rounded up to a
// power of two, threads whose column is >= N idle.  VEC: N is 8, 16, 32 or 64 and rows are 16-byte
// aligned, a thread then owns the eight columns of one 16-byte piece.
template <bool VEC>
__global__ __launch_bounds__(kColsBlock) void rms_cols(const uint16_t *__restrict__ x,
                                                       const uint16_t *__restrict__ w,
                                                       uint16_t *__restrict__ y, int rows, int N,
                                                       int cp, float eps, int rows_per_wg,
                                                       const float *__restrict__ sq,
                                                       int sq_blocks) {
  __shared__ float part[kColsWaves][kMaxCols];
  __shared__ float inv[kMaxCols];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  constexpr int W = VEC ? 8 : 1;           // columns a thread owns
  const int tpr = cp / W;                  // threads per row
  const int col = (threadIdx.x % tpr) * W;
  const int r0 = threadIdx.x / tpr;
  const int rstep = kColsBlock / tpr;
  const bool live = col < N;
  // The first row this thread writes out (its only one at 5120 rows) is requested before the
  // sums, which do not depend on it; rows and columns out of range read element 0 and drop it.
  const int k_lo = blockIdx.x * rows_per_wg;
  const int k_hi = min(rows, k_lo + rows_per_wg);
  const bool first = live && k_lo + r0 < k_hi;
  const size_t at0 = first ? static_cast<size_t>(k_lo + r0) * N + col : 0;
  const uint16_t w0 = w[first ? k_lo + r0 : 0];
  uint4 x0 = make_uint4(0, 0, 0, 0);
  if constexpr (VEC) {
    x0 = *reinterpret_cast<const uint4 *>(x + at0);
  } else {
    x0.x = x[at0];
  }
  if (sq != nullptr) {
    // thread t adds the blocks t / N, t / N + 1024 / N, .. of column t % N; the 1024 / N
    // partial sums of a column meet in the 16 rows of part[], folded in a fixed order
    const int scol = threadIdx.x % N;
    const int sub = threadIdx.x / N;
    const int nsub = kColsBlock / N;         // 16 .. 128
    const int fold = nsub / kColsWaves;      // partial sums per row of part[]
    // The loads of 24 blocks (all of a thread's share at 5120 rows) are issued before the
    // first add, every one unconditional: slots past the last block read the thread's first
    // block again and are not added.  As a plain loop the sum was a chain of trips to memory.
    float t = 0.f;
    constexpr int kBatch = 24;
    for (int b0 = sub; b0 < sq_blocks; b0 += kBatch * nsub) {
      float v[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int b = b0 + u * nsub;
        v[u] = sq[static_cast<size_t>(b < sq_blocks ? b : sub) * N + scol];
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (b0 + u * nsub < sq_blocks) {
          t += v[u];
        }
      }
    }
    for (int f = 0; f < fold; ++f) {
      if (sub % fold == f) {
        float *slot = &part[sub / fold][scol];
        *slot = f == 0 ? t : *slot + t;
      }
      __syncthreads();
    }
  } else {
    float ss[W];
#pragma unroll
    for (int i = 0; i < W; ++i) {
      ss[i] = 0.f;
    }
    if (live) {
#pragma unroll 4
      for (int k = r0; k < rows; k += rstep) {
        const uint16_t *p = x + static_cast<size_t>(k) * N + col;
        if (VEC) {
          const uint4 v = *reinterpret_cast<const uint4 *>(p);
          const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float lo = bf16_lo(d[i]);
            const float hi = bf16_hi(d[i]);
            ss[2 * i] = fmaf(lo, lo, ss[2 * i]);
            ss[2 * i + 1] = fmaf(hi, hi, ss[2 * i + 1]);
          }
        } else {
          const float v = bf16_to_f32(*p);
          ss[0] = fmaf(v, v, ss[0]);
        }
      }
    }
    // lanes that share a column sit tpr apart: fold the wavefront down to its first tpr lanes
#pragma unroll
    for (int i = 0; i < W; ++i) {
      for (int off = kWave / 2; off >= tpr; off >>= 1) {
        ss[i] += __shfl_down(ss[i], off, kWave);
      }
    }
    if (lane < tpr) {
#pragma unroll
      for (int i = 0; i < W; ++i) {
        if (lane * W + i < kMaxCols) {
          part[wave][lane * W + i] = ss[i];
        }
      }
    }
    __syncthreads();
  }
  if (static_cast<int>(threadIdx.x) < N) {
    float t = 0.f;
    for (int i = 0; i < kColsWaves; ++i) {
      t += part[i][threadIdx.x];
    }
    inv[threadIdx.x] = rsqrtf(t / static_cast<float>(rows) + eps);
  }
  __syncthreads();
  if (!live) {
    return;
  }
  for (int k = k_lo + r0; k < k_hi; k += rstep) {
    const size_t at = static_cast<size_t>(k) * N + col;
    const bool pre = k == k_lo + r0;  // the row requested at the top
    const float wk = bf16_to_f32(pre ? w0 : w[k]);
    if (VEC) {
      const uint4 v = pre ? x0 : *reinterpret_cast<const uint4 *>(x + at);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = f32_to_bf16((wk * bf16_lo(d[i])) * inv[col + 2 * i]);
        const uint32_t hi = f32_to_bf16((wk * bf16_hi(d[i])) * inv[col + 2 * i + 1]);
        o[i] = lo | (hi << 16);
      }
      *reinterpret_cast<uint4 *>(y + at) = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
      const uint16_t xv = pre ? static_cast<uint16_t>(x0.x) : x[at];
      y[at] = f32_to_bf16((wk * bf16_to_f32(xv)) * inv[col]);
    }
  }
}

// Rotate-half RoPE of the chunk's q and k at positions *start + n, and the cache write.
// q, k, v are feature-major [heads*hd, N]; q_out is token-major [N, n_q*hd] (what the
// attention reads); the caches are [max_seq, n_kv, hd].  grid.x = head (q heads first, then
// kv heads); a thread takes one token and eight consecutive dims d0 .. d0+7 of the lower
// half plus their partners d0+half ..: lanes run along the tokens, so the reads of a row are
// contiguous, and every store is a 16-byte vector of one token's row.  VEC needs hd % 16 == 0
// and 16-byte aligned outputs and tables; otherwise one pair of dims per thread.
template <bool VEC>
__global__ __launch_bounds__(256) void rope_kv_cols(const uint16_t *__restrict__ q,
                                                    const uint16_t *__restrict__ k,
                                                    const uint16_t *__restrict__ v,
                                                    uint16_t *__restrict__ q_out,
                                                    uint16_t *__restrict__ k_cache,
                                                    uint16_t *__restrict__ v_cache,
                                                    const uint16_t *__restrict__ cos,
                                                    const uint16_t *__restrict__ sin,
                                                    const int64_t *__restrict__ start, int N,
                                                    int n_q, int n_kv, int hd, int max_seq) {
  const long long s0 = *start;
  const int hid = blockIdx.x;
  const bool is_q = hid < n_q;
  const int head = is_q ? hid : hid - n_q;
  const uint16_t *src = (is_q ? q : k) + static_cast<size_t>(head) * hd * N;
  const uint16_t *vsrc = v + static_cast<size_t>(is_q ? 0 : head) * hd * N;
  const int half = hd / 2;
  constexpr int W = VEC ? 8 : 1;  // dims of each half a thread rotates
  const int items = (half / W) * N;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < items; i += gridDim.y * blockDim.x) {
    const int d0 = (i / N) * W;
    const int n = i % N;
    const long long p = s0 + n;
    if (p < 0 || p >= max_seq) {
      continue;
    }
    const uint16_t *c = cos + static_cast<size_t>(p) * hd;
    const uint16_t *sn = sin + static_cast<size_t>(p) * hd;
    // Every load of the item is issued before the first rotation, and none sits under a
    // branch (q heads read v's head 0, a valid address, and drop it): a load inside a
    // conditional is waited for where the conditional ends, which made an item a chain of
    // two dozen trips to memory.
    uint16_t t0[W], t1[W], c0[W], c1[W], s0v[W], s1v[W], vlo[W], vhi[W];
    if constexpr (VEC) {
      // eight consecutive dims of a table row are one 16-byte vector
      auto get8 = [](const uint16_t *src8, uint16_t (&dst)[W]) {
        const uint4 t = *reinterpret_cast<const uint4 *>(src8);
        const uint32_t d4[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int e = 0; e < W; ++e) {
          dst[e] = static_cast<uint16_t>(d4[e >> 1] >> (16 * (e & 1)));
        }
      };
      get8(c + d0, c0);
      get8(c + d0 + half, c1);
      get8(sn + d0, s0v);
      get8(sn + d0 + half, s1v);
    } else {
      c0[0] = c[d0];
      c1[0] = c[d0 + half];
      s0v[0] = sn[d0];
      s1v[0] = sn[d0 + half];
    }
#pragma unroll
    for (int e = 0; e < W; ++e) {
      const int d = d0 + e;
      t0[e] = src[static_cast<size_t>(d) * N + n];
      t1[e] = src[static_cast<size_t>(d + half) * N + n];
      vlo[e] = vsrc[static_cast<size_t>(d) * N + n];
      vhi[e] = vsrc[static_cast<size_t>(d + half) * N + n];
    }
    uint16_t lo[W], hi[W];
#pragma unroll
    for (int e = 0; e < W; ++e) {
      const float a0 = bf16_to_f32(t0[e]);
      const float a1 = bf16_to_f32(t1[e]);
      lo[e] = f32_to_bf16(a0 * bf16_to_f32(c0[e]) + (-a1) * bf16_to_f32(s0v[e]));
      hi[e] = f32_to_bf16(a1 * bf16_to_f32(c1[e]) + a0 * bf16_to_f32(s1v[e]));
    }
    auto put = [](uint16_t *dst, const uint16_t (&val)[W]) {
      if constexpr (VEC) {
        *reinterpret_cast<uint4 *>(dst) = make_uint4(
            val[0] | (static_cast<uint32_t>(val[1]) << 16), val[2] | (static_cast<uint32_t>(val[3]) << 16),
            val[4] | (static_cast<uint32_t>(val[5]) << 16), val[6] | (static_cast<uint32_t>(val[7]) << 16));
      } else {
        dst[0] = val[0];
      }
    };
    if (is_q) {
      uint16_t *dst = q_out + (static_cast<size_t>(n) * n_q + head) * hd;
      put(dst + d0, lo);
      put(dst + d0 + half, hi);
    } else {
      const size_t off = (static_cast<size_t>(p) * n_kv + head) * hd;
      put(k_cache + off + d0, lo);
      put(k_cache + off + d0 + half, hi);
      put(v_cache + off + d0, vlo);
      put(v_cache + off + d0 + half, vhi);
    }
  }
}

// y = silu(gate) * up elementwise (bf16 in, fp32 math, bf16 out).
__global__ __launch_bounds__(256) void swiglu_elems(const uint16_t *__restrict__ g,
                                                    const uint16_t *__restrict__ u,
                                                    uint16_t *__restrict__ y, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < count) {
    const float a = bf16_to_f32(g[i]);
    // the gate product is rounded to bf16 before the multiply, as two separate ops would
    const float act = bf16_to_f32(f32_to_bf16(a / (1.f + expf(-a))));
    y[i] = f32_to_bf16(act * bf16_to_f32(u[i]));
  }
}

// Residual add and/or per-row bias on feature-major data, each sum rounded to bf16 as the
// separate torch adds of the reference round: with a, y = y + (a [+ bias]); without, y += bias.
__global__ __launch_bounds__(256) void add_cols(uint16_t *__restrict__ y,
                                                const uint16_t *__restrict__ a,
                                                const uint16_t *__restrict__ bias, int rows, int N) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < static_cast<int64_t>(rows) * N) {
    const float b = bias != nullptr ? bf16_to_f32(bias[i / N]) : 0.f;
    float v = bf16_to_f32(y[i]);
    if (a != nullptr) {
      float t = bf16_to_f32(a[i]);
      if (bias != nullptr) {
        t = bf16_to_f32(f32_to_bf16(t + b));
      }
      v += t;
    } else {
      v += b;
    }
    y[i] = f32_to_bf16(v);
  }
}

}  // namespace
}  // namespace chr

using namespace chr;

namespace chr {
namespace {

int rms_cols_launch(const void *x, const void *w, void *y, int32_t rows, int32_t N, float eps,
                    const float *sq, int32_t sq_blocks, void *stream) {
  if (x == nullptr || w == nullptr || y == nullptr) {
    return -1;
  }
  if (rows < 1) {
    return -3;
  }
  if (N < 1 || N > kMaxCols) {
    return -2;
  }
  if (sq != nullptr && (kColsBlock % N != 0 || kColsBlock / N < kColsWaves || sq_blocks < 1)) {
    return -2;
  }
  const bool vec = (N == 8 || N == 16 || N == 32 || N == 64) && aligned16(x) && aligned16(y);
  int cp = 1;
  while (cp < N) {
    cp <<= 1;
  }
  // enough workgroups to spread the write-out, few enough that the redundant read stays cheap
  const int wgs = max(1, min(64, rows / 64));
  const int rows_per_wg = (rows + wgs - 1) / wgs;
  const dim3 grid(static_cast<unsigned>((rows + rows_per_wg - 1) / rows_per_wg));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec) {
    rms_cols<true><<<grid, dim3(kColsBlock), 0, st>>>(
        static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(w),
        static_cast<uint16_t *>(y), rows, N, cp, eps, rows_per_wg, sq, sq_blocks);
  } else {
    rms_cols<false><<<grid, dim3(kColsBlock), 0, st>>>(
        static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(w),
        static_cast<uint16_t *>(y), rows, N, cp, eps, rows_per_wg, sq, sq_blocks);
  }
  return launch_rc();
}

}  // namespace
}  // namespace chr

extern "C" int chr_dv2_rms_cols(const void *x, const void *w, void *y, int32_t rows, int32_t N,
                                float eps, void *stream) {
  return rms_cols_launch(x, w, y, rows, N, eps, nullptr, 0, stream);
}

extern "C" int chr_dv2_rms_cols_sq(const void *x, const void *w, void *y, int32_t rows, int32_t N,
                                   float eps, const float *sq, int32_t sq_blocks, void *stream) {
  if (sq == nullptr) {
    return -1;
  }
  return rms_cols_launch(x, w, y, rows, N, eps, sq, sq_blocks, stream);
}

extern "C" int chr_dv2_rope_kv_cols(const void *q, const void *k, const void *v, void *q_out,
                                    void *k_cache, void *v_cache, const void *cos,
                                    const void *sin, const void *start, int32_t N, int32_t n_q,
                                    int32_t n_kv, int32_t hd, int32_t max_seq, void *stream) {
  if (q == nullptr || k == nullptr || v == nullptr || q_out == nullptr || k_cache == nullptr ||
      v_cache == nullptr || cos == nullptr || sin == nullptr || start == nullptr) {
    return -1;
  }
  if (n_q < 1 || n_kv < 1 || hd < 2 || (hd & 1) != 0 || max_seq < 1) {
    return -3;
  }
  if (N < 1 || N > kMaxCols) {
    return -2;
  }
  const bool vec = (hd % 16) == 0 && aligned16(q_out) && aligned16(k_cache) && aligned16(v_cache) &&
                   aligned16(cos) && aligned16(sin);
  const int items = (hd / 2 / (vec ? 8 : 1)) * N;
  const dim3 grid(static_cast<unsigned>(n_q + n_kv), static_cast<unsigned>((items + 255) / 256));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec) {
    rope_kv_cols<true><<<grid, dim3(256), 0, st>>>(
        static_cast<const uint16_t *>(q), static_cast<const uint16_t *>(k),
        static_cast<const uint16_t *>(v), static_cast<uint16_t *>(q_out),
        static_cast<uint16_t *>(k_cache), static_cast<uint16_t *>(v_cache),
        static_cast<const uint16_t *>(cos), static_cast<const uint16_t *>(sin),
        static_cast<const int64_t *>(start), N, n_q, n_kv, hd, max_seq);
  } else {
    rope_kv_cols<false><<<grid, dim3(256), 0, st>>>(
        static_cast<const uint16_t *>(q), static_cast<const uint16_t *>(k),
        static_cast<const uint16_t *>(v), static_cast<uint16_t *>(q_out),
        static_cast<uint16_t *>(k_cache), static_cast<uint16_t *>(v_cache),
        static_cast<const uint16_t *>(cos), static_cast<const uint16_t *>(sin),
        static_cast<const int64_t *>(start), N, n_q, n_kv, hd, max_seq);
  }
  return launch_rc();
}

extern "C" int chr_dv2_swiglu_elems(const void *gate, const void *up, void *y, int64_t count,
                                    void *stream) {
  if (gate == nullptr || up == nullptr || y == nullptr) {
    return -1;
  }
  if (count < 1) {
    return -3;
  }
  swiglu_elems<<<dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0,
                 static_cast<hipStream_t>(stream)>>>(static_cast<const uint16_t *>(gate),
                                                      static_cast<const uint16_t *>(up),
                                                      static_cast<uint16_t *>(y), count);
  return launch_rc();
}

extern "C" int chr_dv2_add_cols(void *y, const void *a, const void *bias, int32_t rows, int32_t N,
                                void *stream) {
  if (y == nullptr || (a == nullptr && bias == nullptr)) {
    return -1;
  }
  if (rows < 1 || N < 1) {
    return -3;
  }
  const int64_t count = static_cast<int64_t>(rows) * N;
  add_cols<<<dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0,
             static_cast<hipStream_t>(stream)>>>(static_cast<uint16_t *>(y),
                                                  static_cast<const uint16_t *>(a),
                                                  static_cast<const uint16_t *>(bias), rows, N);
  return launch_rc();
}

// N=1 NF4 GEMV family for gfx950 (MI355X): plain / residual-add, fused q-k-v,
// fused SwiGLU, and RMSNorm.  Replaces the entry points of
// gpu/nf4/nf4_gemv.cu:790-924, 996-1011.
//
// Row streaming.  A workgroup is four wavefronts of 64 lanes; every wavefront
// owns R weight rows and walks the whole K axis of each.  Lane l reads the
// 16-byte chunk l + 64*j of a row (32 codes, half a scale group), so one
// wavefront load instruction covers 1 KiB of contiguous packed bytes.  The K
// remainder that does not fill 64 such chunks is read as 8-byte half chunks, so
// K = 5120 (160 chunks) costs 2 + 1 steps, not 3.  The R rows of a wavefront
// share the activation registers: x is read and widened to fp32 once per step.
//
// The 16 codebook levels sit at LDS address 0 as 16 consecutive dwords: 16
// distinct addresses in 16 distinct banks, so 64 lanes with arbitrary codes
// never conflict.  A lookup address is one VALU op per code (a byte-select AND);
// lookups of the next packed dword are issued before the FMAs of the current
// one.  The per-group scale multiplies each 32-term partial once.
//
// x is read straight from global memory (it is small and L2-resident).  Only a
// ragged K or the fused RMSNorm make the workgroup stage a bf16 copy in LDS
// first (zero past K, normalised and rounded as a separate RMSNorm launch would).
//
// Numerics: weight = fp32 LUT * fp32(scale) never rounded below fp32, x widened
// bf16->fp32, fp32 accumulation, residual / bias added in fp32, one bf16
// rounding at the store (gpu/nf4/nf4_gemv.cu:70-101, 217-245).

#include "nf4_common.h"

#include <algorithm>
#include <cstdlib>

namespace chr {
namespace {

constexpr int kMaxWaves = 16;  // wavefronts per workgroup, upper bound

// Static LDS of the GEMV kernels.  The codebook comes first so that its LDS
// address is 0 and a lookup address is just 4*code.
struct GemvLds {
  float lut[16];
  float part[kMaxWaves];
  float ksum[kMaxWaves][4];  // K-split: per-wavefront partial dot products of a row group
};

__device__ __forceinline__ float fma8(const Levels8 &v, const float *xf, float acc) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    acc = fmaf(v.l[j], xf[j], acc);
  }
  return acc;
}

__device__ __forceinline__ float dot8(uint32_t w, const float4 xa, const float4 xb,
                                      const float *lut, float acc) {
  const Levels8 v = lookup8(w, lut);
  const float xf[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
  return fma8(v, xf, acc);
}

struct StreamArgs {
  // up to three row segments sharing x (one for a plain GEMV, three for q/k/v)
  const uint8_t *packed[3];
  const uint16_t *scale[3];
  uint16_t *y[3];
  const uint16_t *add[3];  // optional residual / bias per segment, bf16 [M]
  int M[3];
  int groups[3];  // wavefront-sized row groups of each segment
  int ksplit;     // 1, or > 1: the wavefronts of a workgroup share one row group along K
  // x is not given but merged, while it is staged, from the softmax states that
  // attn_parts workgroups per head left: {m, l, 0, 0, o[attn_hd]} each (K = heads*attn_hd)
  const float *attn_state;
  int attn_parts, attn_hd;
  // second matrix of a SwiGLU pair (segment 0 only)
  const uint8_t *packed2;
  const uint16_t *scale2;
  const uint16_t *x;
  const uint16_t *rms_w;  // optional, bf16 [K]
  int K, K_pad;
  float rms_eps;
};

// Sum of a value over the whole workgroup, the same in every thread.
__device__ __forceinline__ float block_sum(float v, float *part) {
  v = wave_sum(v);
  const int waves = blockDim.x >> 6;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    part[threadIdx.x >> 6] = v;
  }
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < waves; ++w) {
    s += part[w];
  }
  __syncthreads();
  return s;
}

// ---- activations staged in LDS ------------------------------------------------------
// A "piece" is 8 consecutive activations (16 bytes of bf16).  In the steps where every
// lane holds a 16-byte chunk of weights, lane l of step j needs pieces 4c..4c+3 of chunk
// c = 64j + l; they are stored as [j][q][l] so that one ds_read_b128 of the wavefront
// covers 64 consecutive pieces (no bank conflicts).  The 8-byte tail chunks need two
// pieces each and are stored as [step][q][l] the same way after the full steps.
__host__ __device__ inline int x_pieces(int K_pad) {
  const int chunks = K_pad >> 5;
  const int nfull = chunks >> 6;
  const int tail_half = (chunks & 63) * 2;
  return nfull * 256 + ((tail_half + 63) >> 6) * 128;
}

__device__ __forceinline__ int x_slot(int piece, int nfull) {
  const int full = nfull << 8;
  if (piece < full) {
    const int c = piece >> 2, q = piece & 3;
    return ((c >> 6) << 8) + (q << 6) + (c & 63);
  }
  const int t = piece - full;
  const int h = t >> 1, q = t & 1;
  return full + ((h >> 6) << 7) + (q << 6) + (h & 63);
}

// Fill the LDS copy: zero for k in [K, K_pad) and for unused slots.  With rms_w the
// value stored is bf16( (w*x) * rsqrt(mean(x^2)+eps) ), i.e. what a separate RMSNorm
// launch would have handed over (gpu/nf4/nf4_gemv.cu:264-289).  Used for a ragged K
// and for the fused RMSNorm.
// x piece i (8 consecutive dims of one head) merged from the per-part softmax states:
// x = sum_p e^{m_p - M} o_p / sum_p e^{m_p - M} l_p, rounded to bf16 as the attention
// launch itself would have stored it.  An empty part has m = -1e30, l = 0: weight zero.
__device__ __forceinline__ uint4 merged_attn_piece(const StreamArgs &a, int i) {
  constexpr int kBatch = 8;  // parts whose states are fetched together (one memory round trip)
  const int hd = a.attn_hd;
  const int k = i << 3;
  const int head = k / hd;
  const int d = k - head * hd;
  const float *st = a.attn_state + static_cast<size_t>(head) * a.attn_parts * (hd + 4);
  float mx = -1e30f;
  float l = 0.f;
  float o[8] = {};
  for (int p0 = 0; p0 < a.attn_parts; p0 += kBatch) {
    float2 ml[kBatch];
    float4 lo[kBatch], hi[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const bool on = p0 + j < a.attn_parts;
      const float *sp = st + (on ? p0 + j : p0) * (hd + 4);
      ml[j] = *reinterpret_cast<const float2 *>(sp);
      lo[j] = *reinterpret_cast<const float4 *>(sp + 4 + d);
      hi[j] = *reinterpret_cast<const float4 *>(sp + 8 + d);
      if (!on) {
        ml[j] = make_float2(-1e30f, 0.f);
      }
    }
    float bm = mx;
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      bm = fmaxf(bm, ml[j].x);
    }
    const float keep = __expf(mx - bm);  // rescale what earlier batches added
    l *= keep;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      o[e] *= keep;
    }
    mx = bm;
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const float w = __expf(ml[j].x - mx);
      l = fmaf(w, ml[j].y, l);
      o[0] = fmaf(w, lo[j].x, o[0]);
      o[1] = fmaf(w, lo[j].y, o[1]);
      o[2] = fmaf(w, lo[j].z, o[2]);
      o[3] = fmaf(w, lo[j].w, o[3]);
      o[4] = fmaf(w, hi[j].x, o[4]);
      o[5] = fmaf(w, hi[j].y, o[5]);
      o[6] = fmaf(w, hi[j].z, o[6]);
      o[7] = fmaf(w, hi[j].w, o[7]);
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  uint32_t r[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t lo16 = f32_to_bf16(o[2 * q] * inv);
    const uint32_t hi16 = f32_to_bf16(o[2 * q + 1] * inv);
    r[q] = lo16 | (hi16 << 16);
  }
  return make_uint4(r[0], r[1], r[2], r[3]);
}

__device__ __forceinline__ void stage_x(const StreamArgs &a, uint4 *xs, float *part) {
  if (a.attn_state != nullptr) {
    const int nfull_a = (a.K_pad >> 5) >> 6;
    for (int i = threadIdx.x; i < (a.K_pad >> 3); i += blockDim.x) {
      xs[x_slot(i, nfull_a)] = merged_attn_piece(a, i);
    }
    const int full = nfull_a << 8;
    const int tail_half = ((a.K_pad >> 5) & 63) * 2;
    for (int i = full + threadIdx.x; i < x_pieces(a.K_pad); i += blockDim.x) {
      const int h = (((i - full) >> 7) << 6) + (i & 63);
      if (h >= tail_half) {
        xs[i] = make_uint4(0, 0, 0, 0);
      }
    }
    __syncthreads();
    return;
  }
  constexpr int kKeep = 4;  // 16-byte vectors of x a thread keeps between the two passes
  const int nfull = (a.K_pad >> 5) >> 6;
  const int slots = x_pieces(a.K_pad);
  const int nvec = a.K_pad >> 3;
  const bool vec_ok = (a.K & 7) == 0 && aligned16(a.x) &&
                      (a.rms_w == nullptr || aligned16(a.rms_w)) &&
                      nvec <= kKeep * static_cast<int>(blockDim.x);
  // Slots of the last tail step that no piece maps to (lanes past the end of the row).
  {
    const int full = nfull << 8;
    const int tail_half = ((a.K_pad >> 5) & 63) * 2;
    for (int i = full + threadIdx.x; i < slots; i += blockDim.x) {
      const int h = (((i - full) >> 7) << 6) + (i & 63);
      if (h >= tail_half) {
        xs[i] = make_uint4(0, 0, 0, 0);
      }
    }
  }
  if (vec_ok) {
    // x and the norm weights are requested together: one memory round trip, not two.
    uint4 v[kKeep], g[kKeep];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      v[j] = make_uint4(0, 0, 0, 0);
      g[j] = make_uint4(0, 0, 0, 0);
      if (i * 8 < a.K) {
        v[j] = reinterpret_cast<const uint4 *>(a.x)[i];
        if (a.rms_w != nullptr) {
          g[j] = reinterpret_cast<const uint4 *>(a.rms_w)[i];
        }
      }
    }
    float inv = 1.f;
    if (a.rms_w != nullptr) {
#pragma unroll
      for (int j = 0; j < kKeep; ++j) {
        const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          ss = fmaf(bf16_lo(u[q]), bf16_lo(u[q]), ss);
          ss = fmaf(bf16_hi(u[q]), bf16_hi(u[q]), ss);
        }
      }
      ss = block_sum(ss, part);
      inv = rsqrtf(ss / static_cast<float>(a.K) + a.rms_eps);
    }
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i < nvec) {
        uint4 o = v[j];
        if (a.rms_w != nullptr && i * 8 < a.K) {
          const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
          const uint32_t gw[4] = {g[j].x, g[j].y, g[j].z, g[j].w};
          uint32_t r[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t lo = f32_to_bf16((bf16_lo(gw[q]) * bf16_lo(u[q])) * inv);
            const uint32_t hi = f32_to_bf16((bf16_hi(gw[q]) * bf16_hi(u[q])) * inv);
            r[q] = lo | (hi << 16);
          }
          o = make_uint4(r[0], r[1], r[2], r[3]);
        }
        xs[x_slot(i, nfull)] = o;
      }
    }
  } else {
    float inv = 1.f;
    if (a.rms_w != nullptr) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < a.K; i += blockDim.x) {
        const float v = bf16_to_f32(a.x[i]);
        ss = fmaf(v, v, ss);
      }
      ss = block_sum(ss, part);
      inv = rsqrtf(ss / static_cast<float>(a.K) + a.rms_eps);
    }
    uint16_t *xh = reinterpret_cast<uint16_t *>(xs);
    for (int i = threadIdx.x; i < a.K_pad; i += blockDim.x) {
      uint16_t v = 0;
      if (i < a.K) {
        v = a.x[i];
        if (a.rms_w != nullptr) {
          v = f32_to_bf16((bf16_to_f32(a.rms_w[i]) * bf16_to_f32(v)) * inv);
        }
      }
      xh[(x_slot(i >> 3, nfull) << 3) + (i & 7)] = v;
    }
  }
  __syncthreads();
}

__device__ __forceinline__ void widen8(const uint4 v, float *xf) {
  xf[0] = bf16_lo(v.x);
  xf[1] = bf16_hi(v.x);
  xf[2] = bf16_lo(v.y);
  xf[3] = bf16_hi(v.y);
  xf[4] = bf16_lo(v.z);
  xf[5] = bf16_hi(v.z);
  xf[6] = bf16_lo(v.w);
  xf[7] = bf16_hi(v.w);
}

// NW packed dwords per row against the same NW*8 activations, R rows.  The
// lookups of dword i+1 are issued before the FMAs of dword i, so LDS latency is
// covered by arithmetic inside the wavefront.
template <int R, int NW>
__device__ __forceinline__ void rows_step(const uint32_t (&w)[R][NW], const float *xf,
                                          const uint16_t (&sc)[R], const float *lut,
                                          float (&acc)[R]) {
  constexpr int N = R * NW;
  float p[R] = {};
  Levels8 cur = lookup8(w[0][0], lut);
#pragma unroll
  for (int i = 1; i < N; ++i) {
    const Levels8 nxt = lookup8(w[i / NW][i % NW], lut);
    __builtin_amdgcn_sched_barrier(0);
    p[(i - 1) / NW] = fma8(cur, xf + 8 * ((i - 1) % NW), p[(i - 1) / NW]);
    __builtin_amdgcn_sched_barrier(0);
    cur = nxt;
  }
  p[R - 1] = fma8(cur, xf + 8 * (NW - 1), p[R - 1]);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = fmaf(f16_to_f32(sc[r]), p[r], acc[r]);
  }
}

// One wavefront, R weight rows sharing x.  x4 points at the activations as 16-byte
// pieces: K_pad/8 of them in global memory (XL == false), or the LDS copy made by
// stage_x in its [step][q][lane] order (XL == true).
template <int R, bool XL>
__device__ __forceinline__ void rows_dot(const uint8_t *const (&prow)[R],
                                         const uint16_t *const (&srow)[R], const uint4 *x4,
                                         int K_pad, const float *lut, int lane,
                                         float (&acc)[R], int t0 = 0, int tstep = 1) {
  const int chunks = K_pad >> 5;            // 16-byte chunks per row
  const int nfull = chunks >> 6;            // steps where all 64 lanes hold a chunk
  const int tail_half = (chunks & 63) * 2;  // 8-byte half chunks after them
  const int nsteps = nfull + ((tail_half + kWave - 1) >> 6);
  const int base_half = nfull << 7;         // first half chunk of the tail

  // Steps t0, t0 + tstep, ..: all of them for a wavefront that owns its rows, every
  // tstep-th one when the wavefronts of a workgroup share a row group along K.
  for (int t = t0; t < nsteps; t += tstep) {
    if (t < nfull) {
      const int c = (t << 6) + lane;
      uint32_t w[R][4];
      uint16_t sc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint4 v = *(reinterpret_cast<const uint4 *>(prow[r]) + c);
        w[r][0] = v.x;
        w[r][1] = v.y;
        w[r][2] = v.z;
        w[r][3] = v.w;
        sc[r] = srow[r][c >> 1];
      }
      const uint4 *xp = XL ? x4 + (t << 8) + lane : x4 + (c << 2);
      constexpr int xq = XL ? 64 : 1;
      const uint4 x0 = xp[0], x1 = xp[xq], x2 = xp[2 * xq], x3 = xp[3 * xq];
      float xf[32];
      widen8(x0, xf);
      widen8(x1, xf + 8);
      widen8(x2, xf + 16);
      widen8(x3, xf + 24);
      rows_step<R, 4>(w, xf, sc, lut, acc);
    } else {
      const int h0 = (t - nfull) << 6;
      const int h = h0 + lane;
      if (h < tail_half) {
        const int hc = base_half + h;  // half-chunk index in the row: 16 weights
        uint32_t w[R][2];
        uint16_t sc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint2 v = *(reinterpret_cast<const uint2 *>(prow[r]) + hc);
          w[r][0] = v.x;
          w[r][1] = v.y;
          sc[r] = srow[r][hc >> 2];
        }
        const uint4 *xp = XL ? x4 + (nfull << 8) + ((h0 >> 6) << 7) + lane : x4 + (hc << 1);
        const uint4 x0 = xp[0], x1 = xp[XL ? 64 : 1];
        float xf[16];
        widen8(x0, xf);
        widen8(x1, xf + 8);
        rows_step<R, 2>(w, xf, sc, lut, acc);
      }
    }
  }
}

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }

// SWIGLU == false: R rows of one segment per wavefront, epilogue y = acc (+ add).
// SWIGLU == true : R/2 gate rows and the matching R/2 up rows per wavefront,
//                  epilogue y = silu(gate) * up from the unrounded fp32 sums.
// XLDS: x is first copied (and optionally RMS-normalised) into LDS.
template <int R, bool SWIGLU, bool XLDS>
__global__ __launch_bounds__(XLDS ? 1024 : 256) void gemv_stream(const StreamArgs a) {
  extern __shared__ uint4 xs[];
  __shared__ GemvLds lds;
  constexpr int U = SWIGLU ? R / 2 : R;  // output rows per wavefront
  const int lane = threadIdx.x & (kWave - 1);
  // The wavefront index is the same in every lane: saying so keeps the row-group and
  // segment arithmetic, and the kernel-argument reads indexed by it, on the scalar unit.
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int waves = blockDim.x >> 6;

  if (threadIdx.x < 16) {
    lds.lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  // Row groups (U rows each) are numbered through the segments.  Without the LDS
  // copy a wavefront takes exactly one group; with it the grid is one workgroup per
  // compute unit and a wavefront walks groups wave*grid + block, + grid*waves, ..,
  // so the copy is made once per compute unit and units stay balanced to one group.
  const int total = a.groups[0] + a.groups[1] + a.groups[2];
  const bool ksplit = !XLDS && !SWIGLU && a.ksplit > 1;
  const int first = XLDS     ? wave * static_cast<int>(gridDim.x) + static_cast<int>(blockIdx.x)
                    : ksplit ? static_cast<int>(blockIdx.x)
                             : static_cast<int>(blockIdx.x) * waves + wave;
  const int stride = static_cast<int>(gridDim.x) * waves;
  const size_t pstride = static_cast<size_t>(a.K_pad >> 1);
  const size_t sstride = static_cast<size_t>(a.K_pad >> 6);

  if constexpr (XLDS) {
    stage_x(a, xs, lds.part);
  } else {
    __syncthreads();
  }

  auto run_group = [&](int grp) {
    int g = grp;
    int seg = 0;
    if (!SWIGLU) {
      if (g >= a.groups[0]) {
        g -= a.groups[0];
        seg = 1;
        if (g >= a.groups[1]) {
          g -= a.groups[1];
          seg = 2;
        }
      }
    }
    const int M = a.M[seg];
    const int row0 = g * U;
    const uint8_t *prow[R];
    const uint16_t *srow[R];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = min(row0 + u, M - 1);  // rows past M are computed, never stored
      prow[u] = a.packed[seg] + r * pstride;
      srow[u] = a.scale[seg] + r * sstride;
      if constexpr (SWIGLU) {
        prow[U + u] = a.packed2 + r * pstride;
        srow[U + u] = a.scale2 + r * sstride;
      }
    }

    float acc[R] = {};
    if constexpr (XLDS) {
      rows_dot<R, true>(prow, srow, static_cast<const uint4 *>(xs), a.K_pad, lds.lut, lane, acc);
    } else {
      rows_dot<R, false>(prow, srow, reinterpret_cast<const uint4 *>(a.x), a.K_pad, lds.lut, lane,
                         acc, ksplit ? wave : 0, ksplit ? waves : 1);
    }

    if constexpr (SWIGLU) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float gsum = wave_sum(acc[u]);
        const float usum = wave_sum(acc[U + u]);
        const int r = row0 + u;
        if (lane == u && r < M) {
          a.y[0][r] = f32_to_bf16(silu(gsum) * usum);
        }
      }
    } else {
      const uint16_t *add = a.add[seg];
      uint16_t *y = a.y[seg];
      float sums[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        sums[u] = wave_sum(acc[u]);
      }
      bool writer = true;
      if (ksplit) {
        // every wavefront of the workgroup holds a partial of the same rows: add them in
        // wavefront order, wavefront 0 finishes
        if (lane == 0) {
#pragma unroll
          for (int u = 0; u < U; ++u) {
            lds.ksum[wave][u] = sums[u];
          }
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float t = 0.f;
          for (int w = 0; w < waves; ++w) {
            t += lds.ksum[w][u];
          }
          sums[u] = t;
        }
        writer = wave == 0;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float s = sums[u];
        const int r = row0 + u;
        if (writer && lane == u && r < M) {
          float v = s;
          if (add != nullptr) {
            v += bf16_to_f32(add[r]);
          }
          y[r] = f32_to_bf16(v);
        }
      }
    }
  };
  if constexpr (XLDS) {
    for (int grp = first; grp < total; grp += stride) {
      run_group(grp);
    }
  } else {
    if (first < total) {
      run_group(first);  // exactly one group per wavefront
    }
  }
}

// ---- RMSNorm -----------------------------------------------------------------
constexpr int kRmsBlock = 1024;

__global__ __launch_bounds__(kRmsBlock) void rms_vec(const uint16_t *__restrict__ x,
                                                     const uint16_t *__restrict__ w,
                                                     uint16_t *__restrict__ y, int n, float eps) {
  __shared__ float part[kRmsBlock / kWave];
  // Up to 8 elements per thread stay in registers (n <= 8192), so x and w are
  // each read once and both loads are in flight before the reduction.
  constexpr int kKeep = 8;
  float xv[kKeep], wv[kKeep];
  float a = 0.f;
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int i = threadIdx.x + j * kRmsBlock;
    xv[j] = i < n ? bf16_to_f32(x[i]) : 0.f;
    wv[j] = i < n ? bf16_to_f32(w[i]) : 0.f;
  }
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    a = fmaf(xv[j], xv[j], a);
  }
  for (int i = threadIdx.x + kKeep * kRmsBlock; i < n; i += kRmsBlock) {
    const float v = bf16_to_f32(x[i]);
    a = fmaf(v, v, a);
  }
  a = wave_sum(a);
  if ((threadIdx.x & (kWave - 1)) == 0) {
    part[threadIdx.x >> 6] = a;
  }
  __syncthreads();
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kRmsBlock / kWave; ++i) {
    sum += part[i];
  }
  const float inv = rsqrtf(sum / static_cast<float>(n) + eps);
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int i = threadIdx.x + j * kRmsBlock;
    if (i < n) {
      y[i] = f32_to_bf16((wv[j] * xv[j]) * inv);
    }
  }
  for (int i = threadIdx.x + kKeep * kRmsBlock; i < n; i += kRmsBlock) {
    y[i] = f32_to_bf16((bf16_to_f32(w[i]) * bf16_to_f32(x[i])) * inv);
  }
}

// ---- launch policy -------------------------------------------------------------
// Rows per wavefront forced by CHR_NF4_GEMV_NR (1|2|4), read on every launch so
// a test or a sweep can change it inside one process; 0 = automatic.
int forced_rows() {
  const char *e = std::getenv("CHR_NF4_GEMV_NR");
  if (e != nullptr && e[0] != '\0') {
    const int n = std::atoi(e);
    if (n == 1 || n == 2 || n == 4) {
      return n;
    }
  }
  return 0;
}

// Rows per wavefront for M output rows: two rows share x and keep registers low
// enough for four wavefronts per SIMD; one row when M is too small to fill 256
// compute units otherwise.
int rows_for_m(int M) {
  const int f = forced_rows();
  if (f > 0) {
    return f;
  }
  if (M >= 32768) {
    return 4;  // long streams (lm_head): the x registers are shared by more rows
  }
  return M >= 4096 ? 2 : 1;
}

// CHR_NF4_GEMV_STAGED=0|1 forces the kernel family (read on every launch); unset = automatic.
int forced_staged() {
  const char *e = std::getenv("CHR_NF4_GEMV_STAGED");
  if (e != nullptr && (e[0] == '0' || e[0] == '1') && e[1] == '\0') {
    return e[0] - '0';
  }
  return -1;
}

constexpr int kThreads = 256;
constexpr int kStagedThreads = 1024;  // workgroup of the kernels that stage x in LDS
constexpr size_t kMaxDynLds = 150 * 1024;

template <typename Kern>
int prep_lds(Kern kern, size_t dyn) {
  if (dyn > kMaxDynLds) {
    return -6;
  }
  if (dyn > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(dyn)) != hipSuccess) {
      (void)hipGetLastError();
      return -6;
    }
  }
  return 0;
}

template <int R, bool SWIGLU>
int launch_stream(StreamArgs &a, int n_seg, hipStream_t st) {
  constexpr int U = SWIGLU ? R / 2 : R;
  int total = 0;
  for (int i = 0; i < 3; ++i) {
    a.groups[i] = i < n_seg ? (a.M[i] + U - 1) / U : 0;
    total += a.groups[i];
  }
  const size_t dyn = static_cast<size_t>(x_pieces(a.K_pad)) * 16;
  const bool must_stage = a.rms_w != nullptr || a.K != a.K_pad || a.attn_state != nullptr;
  const int forced = forced_staged();
  const bool staged = must_stage || (forced == 1 && dyn <= kMaxDynLds);
  if (staged) {
    if (prep_lds(gemv_stream<R, SWIGLU, true>, dyn) != 0) {
      return -6;
    }
    const int waves = kStagedThreads / kWave;
    const int grid = std::min(device_cu_count(), (total + waves - 1) / waves);
    gemv_stream<R, SWIGLU, true><<<dim3(grid), dim3(kStagedThreads), dyn, st>>>(a);
  } else {
    const int waves = kThreads / kWave;
    // Long rows and few of them (a down projection): a wavefront walking a whole row pays
    // the memory latency once per step, so the four wavefronts of a workgroup split the
    // steps of one row group instead.
    const int nsteps = (a.K_pad + 2047) / 2048;
    const bool split = !SWIGLU && nsteps >= 4 && total * 4 <= 16 * device_cu_count() * 4;
    a.ksplit = split ? waves : 1;
    const int grid = split ? total : (total + waves - 1) / waves;
    gemv_stream<R, SWIGLU, false><<<dim3(grid), dim3(kThreads), 0, st>>>(a);
  }
  return launch_rc();
}

int launch_rows(StreamArgs &a, int n_seg, int m_for_policy, hipStream_t st) {
  switch (rows_for_m(m_for_policy)) {
    case 4:
      return launch_stream<4, false>(a, n_seg, st);
    case 2:
      return launch_stream<2, false>(a, n_seg, st);
    default:
      return launch_stream<1, false>(a, n_seg, st);
  }
}

}  // namespace

// Shared with the GEMM entry points, which route N == 1 here.
int gemv_entry(const chr_nf4_dev_t *w, const void *x, void *y, void *stream, const void *add,
               const void *rms_w, float rms_eps) {
  if (w == nullptr || x == nullptr || y == nullptr) {
    return -1;
  }
  if (w->M < 1 || w->K < 1 || w->packed == nullptr || w->scale == nullptr) {
    return -3;
  }
  if (!k_pad_ok(w->K, w->K_pad)) {
    return -4;
  }
  if (!aligned16(w->packed) || !aligned16(x) || !aligned2(w->scale)) {
    return -5;
  }
  StreamArgs a{};
  a.packed[0] = w->packed;
  a.scale[0] = w->scale;
  a.y[0] = static_cast<uint16_t *>(y);
  a.add[0] = static_cast<const uint16_t *>(add);
  a.M[0] = w->M;
  a.x = static_cast<const uint16_t *>(x);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.K = w->K;
  a.K_pad = w->K_pad;
  a.rms_eps = rms_eps;
  return launch_rows(a, 1, w->M, static_cast<hipStream_t>(stream));
}

// y = W @ merge(states) (+ add): the o projection consuming what chr_dv2_attn_parts left.
int gemv_attn_entry(const chr_nf4_dev_t *w, const float *state, int n_q, int hd, int n_parts,
                    void *y, const void *add, void *stream) {
  if (w == nullptr || state == nullptr || y == nullptr) {
    return -1;
  }
  if (w->M < 1 || w->K < 1 || w->packed == nullptr || w->scale == nullptr || n_q < 1 || hd < 8 ||
      (hd & 7) != 0 || n_parts < 1 || n_parts > 64 || w->K != n_q * hd) {
    return -3;
  }
  if (!k_pad_ok(w->K, w->K_pad) || w->K != w->K_pad) {
    return -4;
  }
  if (!aligned16(w->packed) || !aligned16(state) || !aligned2(w->scale)) {
    return -5;
  }
  StreamArgs a{};
  a.packed[0] = w->packed;
  a.scale[0] = w->scale;
  a.y[0] = static_cast<uint16_t *>(y);
  a.add[0] = static_cast<const uint16_t *>(add);
  a.M[0] = w->M;
  a.K = w->K;
  a.K_pad = w->K_pad;
  a.attn_state = state;
  a.attn_parts = n_parts;
  a.attn_hd = hd;
  return launch_rows(a, 1, w->M, static_cast<hipStream_t>(stream));
}

// Launch geometry of the N=1 path, reported by the planner.
int gemv_rows_per_wg(int M, int K_pad) {
  (void)K_pad;
  return (kThreads / kWave) * rows_for_m(M);
}

int gemv_threads_per_wg(int M, int K_pad) {
  (void)M;
  (void)K_pad;
  return kThreads;
}

int gemv_lds_bytes(int K_pad) {
  (void)K_pad;
  return static_cast<int>(sizeof(GemvLds));
}

}  // namespace chr

using namespace chr;

extern "C" int chr_nf4_gemv(const chr_nf4_dev_t *w, const void *x, void *y, void *stream,
                            const void *add, const void *rms_w, float rms_eps) {
  return gemv_entry(w, x, y, stream, add, rms_w, rms_eps);
}

extern "C" int chr_nf4_gemv_qkv(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                                const chr_nf4_dev_t *v, const void *x, void *yq, void *yk,
                                void *yv, const void *bq, const void *bk, const void *bv,
                                void *stream, const void *rms_w, float rms_eps) {
  if (q == nullptr || k == nullptr || v == nullptr || x == nullptr || yq == nullptr ||
      yk == nullptr || yv == nullptr) {
    return -1;
  }
  if (q->M < 1 || k->M < 1 || v->M < 1 || q->K < 1 || q->packed == nullptr ||
      k->packed == nullptr || v->packed == nullptr || q->scale == nullptr ||
      k->scale == nullptr || v->scale == nullptr) {
    return -3;
  }
  if (k->K != q->K || v->K != q->K || k->K_pad != q->K_pad || v->K_pad != q->K_pad) {
    return -3;
  }
  if (!k_pad_ok(q->K, q->K_pad)) {
    return -4;
  }
  if (!aligned16(q->packed) || !aligned16(k->packed) || !aligned16(v->packed) || !aligned16(x)) {
    return -5;
  }
  StreamArgs a{};
  const chr_nf4_dev_t *m[3] = {q, k, v};
  void *ys[3] = {yq, yk, yv};
  const void *bs[3] = {bq, bk, bv};
  for (int i = 0; i < 3; ++i) {
    a.packed[i] = m[i]->packed;
    a.scale[i] = m[i]->scale;
    a.y[i] = static_cast<uint16_t *>(ys[i]);
    a.add[i] = static_cast<const uint16_t *>(bs[i]);
    a.M[i] = m[i]->M;
  }
  a.x = static_cast<const uint16_t *>(x);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.K = q->K;
  a.K_pad = q->K_pad;
  a.rms_eps = rms_eps;
  return launch_rows(a, 3, q->M + k->M + v->M, static_cast<hipStream_t>(stream));
}

extern "C" int chr_nf4_gemv_swiglu(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                                   const void *x, void *y, void *stream, const void *rms_w,
                                   float rms_eps) {
  if (gate == nullptr || up == nullptr || x == nullptr || y == nullptr) {
    return -1;
  }
  if (gate->M < 1 || gate->K < 1 || up->M != gate->M || up->K != gate->K ||
      up->K_pad != gate->K_pad || gate->packed == nullptr || up->packed == nullptr ||
      gate->scale == nullptr || up->scale == nullptr) {
    return -3;
  }
  if (!k_pad_ok(gate->K, gate->K_pad)) {
    return -4;
  }
  if (!aligned16(gate->packed) || !aligned16(up->packed) || !aligned16(x)) {
    return -5;
  }
  StreamArgs a{};
  a.packed[0] = gate->packed;
  a.scale[0] = gate->scale;
  a.packed2 = up->packed;
  a.scale2 = up->scale;
  a.y[0] = static_cast<uint16_t *>(y);
  a.M[0] = gate->M;
  a.x = static_cast<const uint16_t *>(x);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.K = gate->K;
  a.K_pad = gate->K_pad;
  a.rms_eps = rms_eps;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // A gate/up pair is two weight streams per output row.
  if (rows_for_m(2 * gate->M) >= 2) {
    return launch_stream<4, true>(a, 1, st);
  }
  return launch_stream<2, true>(a, 1, st);
}

extern "C" int chr_nf4_rms(const void *x, const void *w, void *y, int32_t n, float eps,
                           void *stream) {
  if (x == nullptr || w == nullptr || y == nullptr) {
    return -1;
  }
  if (n < 1) {
    return -3;
  }
  rms_vec<<<dim3(1), dim3(kRmsBlock), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(w),
      static_cast<uint16_t *>(y), n, eps);
  return launch_rc();
}

// N=1 NF4 GEMV family for gfx950 (MI355X): plain / residual-add, fused q-k-v,
// fused SwiGLU, RMSNorm, plus the codec twins (dequant, embedding-row gather,
// quantise).  Replaces the entry points of gpu/nf4/nf4_gemv.cu:790-1011.
//
// Row-streaming layout.  A workgroup is four 64-lane wavefronts; every
// wavefront owns U consecutive output rows and walks the whole K axis of each.
// Lane l reads the 16-byte chunk l + 64*j of a row (32 codes, half a scale
// group), so one wavefront load instruction covers 1 KiB of contiguous packed
// bytes.  The K remainder that does not fill 64 such chunks is walked in
// 8-byte half chunks, so K = 5120 (160 chunks) costs 2 + 1 steps, not 3.
// The U rows of a wavefront share the activation registers: x is read and
// widened to fp32 once per step and reused by every row.
//
// The 16 codebook levels sit in LDS as 16 consecutive dwords: 16 distinct
// addresses in 16 distinct banks, so 64 lanes with arbitrary codes never
// conflict.  The per-group scale multiplies the 32-term partial once.
//
// Numerics: weight = fp32 LUT * fp32(scale) never rounded below fp32, x widened
// bf16->fp32, fp32 accumulation, residual / bias added in fp32, one bf16
// rounding at the store (gpu/nf4/nf4_gemv.cu:70-101, 217-245).

#include "nf4_common.h"

#include <cstdlib>

namespace chr {
namespace {

constexpr int kWavesPerWG = 4;
constexpr int kBlock = kWavesPerWG * kWave;

// Static LDS of every GEMV kernel.  The codebook comes first so that its LDS
// address is 0 and a lookup address is just 4*code.
struct GemvLds {
  float lut[16];
  float part[kWavesPerWG];
};

__device__ __forceinline__ void load_lut_lds(float *lut) {
  if (threadIdx.x < 16) {
    lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  __syncthreads();
}

// lut is an LDS array of 16 floats; off is a byte offset in {0,4,..,60}.
__device__ __forceinline__ float lut_at(const float *lut, uint32_t off) {
  return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(lut) + off);
}

// (byte J of w) & mask in one VALU op: the sub-dword source select of gfx9
// SDWA picks the byte, so no separate shift or bit-field extract is needed.
template <int J>
__device__ __forceinline__ uint32_t and_byte(uint32_t w, uint32_t mask) {
  uint32_t r;
  if constexpr (J == 0) {
    asm("v_and_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0 "
        "src1_sel:DWORD"
        : "=v"(r)
        : "v"(w), "v"(mask));
  } else if constexpr (J == 1) {
    asm("v_and_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1 "
        "src1_sel:DWORD"
        : "=v"(r)
        : "v"(w), "v"(mask));
  } else if constexpr (J == 2) {
    asm("v_and_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2 "
        "src1_sel:DWORD"
        : "=v"(r)
        : "v"(w), "v"(mask));
  } else {
    asm("v_and_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3 "
        "src1_sel:DWORD"
        : "=v"(r)
        : "v"(w), "v"(mask));
  }
  return r;
}

// Eight codes of one dword against eight fp32 activations.  In (w << 2) byte j
// carries 4*code(2j) in bits 2..5; in (w >> 2) byte j carries 4*code(2j+1)
// there.  Masking a selected byte with 0x3C is the LDS byte offset of the
// level.  The eight lookups are issued together, then the eight FMAs.
__device__ __forceinline__ float dot8(uint32_t w, const float *xf, const float *lut,
                                      float acc) {
  const uint32_t ev = w << 2;
  const uint32_t od = w >> 2;
  const uint32_t mask = 0x3Cu;
  float lv[8];
  lv[0] = lut_at(lut, and_byte<0>(ev, mask));
  lv[1] = lut_at(lut, and_byte<0>(od, mask));
  lv[2] = lut_at(lut, and_byte<1>(ev, mask));
  lv[3] = lut_at(lut, and_byte<1>(od, mask));
  lv[4] = lut_at(lut, and_byte<2>(ev, mask));
  lv[5] = lut_at(lut, and_byte<2>(od, mask));
  lv[6] = lut_at(lut, and_byte<3>(ev, mask));
  lv[7] = lut_at(lut, and_byte<3>(od, mask));
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    acc = fmaf(lv[j], xf[j], acc);
  }
  return acc;
}

// Widen 8 bf16 (one uint4) to fp32.
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

template <typename T>
__device__ __forceinline__ T ldg(const T *p) {
  return *p;
}

// One wavefront, R weight rows that share x.  rows[r]/scales[r] point at the
// start of row r's packed bytes / scales.  K_pad is a multiple of 64 and the
// K axis is fully valid (K == K_pad); acc[r] receives the lane partials.
template <int R>
__device__ __forceinline__ void rows_dot(const uint8_t *const (&prow)[R],
                                         const uint16_t *const (&srow)[R],
                                         const uint16_t *__restrict__ x, int K_pad,
                                         const float *lut, int lane, float (&acc)[R]) {
  const int chunks = K_pad >> 5;  // 16-byte chunks per row
  const int nfull = chunks >> 6;  // steps where all 64 lanes hold a chunk
  const int tail_half = (chunks & 63) * 2;  // 8-byte half chunks after them

  for (int j = 0; j < nfull; ++j) {
    const int c = (j << 6) + lane;
    uint4 pk[R];
    uint16_t sc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      pk[r] = ldg(reinterpret_cast<const uint4 *>(prow[r]) + c);
      sc[r] = ldg(srow[r] + (c >> 1));
    }
    const uint4 *xp = reinterpret_cast<const uint4 *>(x) + (c << 2);
    const uint4 x0 = ldg(xp), x1 = ldg(xp + 1), x2 = ldg(xp + 2), x3 = ldg(xp + 3);
    float xf[32];
    widen8(x0, xf);
    widen8(x1, xf + 8);
    widen8(x2, xf + 16);
    widen8(x3, xf + 24);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float p = 0.f;
      p = dot8(pk[r].x, xf, lut, p);
      p = dot8(pk[r].y, xf + 8, lut, p);
      p = dot8(pk[r].z, xf + 16, lut, p);
      p = dot8(pk[r].w, xf + 24, lut, p);
      acc[r] = fmaf(f16_to_f32(sc[r]), p, acc[r]);
    }
  }

  const int base_half = nfull << 7;  // first half chunk of the tail
  for (int h0 = 0; h0 < tail_half; h0 += kWave) {
    const int h = h0 + lane;
    if (h < tail_half) {
      const int hc = base_half + h;  // half-chunk index in the row: 16 weights
      uint2 pk[R];
      uint16_t sc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        pk[r] = ldg(reinterpret_cast<const uint2 *>(prow[r]) + hc);
        sc[r] = ldg(srow[r] + (hc >> 2));
      }
      const uint4 *xp = reinterpret_cast<const uint4 *>(x) + (hc << 1);
      const uint4 x0 = ldg(xp), x1 = ldg(xp + 1);
      float xf[16];
      widen8(x0, xf);
      widen8(x1, xf + 8);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float p = 0.f;
        p = dot8(pk[r].x, xf, lut, p);
        p = dot8(pk[r].y, xf + 8, lut, p);
        acc[r] = fmaf(f16_to_f32(sc[r]), p, acc[r]);
      }
    }
  }
}

// Ragged K (K < K_pad) or an activation vector that lives in LDS: one dword
// (8 codes) per lane per step, every activation fetched under a k < K guard so
// that padding codes never meet a live x.  Slow path; model shapes never use it
// on global x.
template <int R, typename XPtr>
__device__ __forceinline__ void rows_dot_guarded(const uint8_t *const (&prow)[R],
                                                 const uint16_t *const (&srow)[R], XPtr x,
                                                 int K, int K_pad, const float *lut, int lane,
                                                 float (&acc)[R]) {
  const int dwords = K_pad >> 3;
  for (int d = lane; d < dwords; d += kWave) {
    float xf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = (d << 3) + i;
      xf[i] = k < K ? bf16_to_f32(x[k]) : 0.f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t w = ldg(reinterpret_cast<const uint32_t *>(prow[r]) + d);
      const float s = f16_to_f32(ldg(srow[r] + (d >> 3)));
      acc[r] = fmaf(s, dot8(w, xf, lut, 0.f), acc[r]);
    }
  }
}

// RMSNorm of x into LDS as bf16 (the rounding the standalone RMS kernel makes),
// for the optional rms_w argument of the GEMV entry points
// (gpu/nf4/nf4_gemv.cu:264-289).  part: kWavesPerWG floats of LDS.
__device__ void rms_to_lds(const uint16_t *__restrict__ x, const uint16_t *__restrict__ rms_w,
                           int K, float eps, uint16_t *xh, float *part) {
  float a = 0.f;
  for (int i = threadIdx.x; i < K; i += kBlock) {
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
  for (int w = 0; w < kWavesPerWG; ++w) {
    sum += part[w];
  }
  const float inv = rsqrtf(sum / static_cast<float>(K) + eps);
  for (int i = threadIdx.x; i < K; i += kBlock) {
    xh[i] = f32_to_bf16((bf16_to_f32(rms_w[i]) * bf16_to_f32(x[i])) * inv);
  }
  __syncthreads();
}

enum : int { kXGlobalFast = 0, kXGlobalGuarded = 1, kXLds = 2 };

struct GemvArgs {
  const uint8_t *packed;
  const uint16_t *scale;
  const uint16_t *x;
  uint16_t *y;
  const uint16_t *add;    // optional residual / bias, bf16 [M]
  const uint16_t *rms_w;  // optional, bf16 [K]
  int M, K, K_pad;
  float rms_eps;
};

template <int U, int XMODE>
__global__ __launch_bounds__(kBlock) void gemv_rows(const GemvArgs a) {
  extern __shared__ uint16_t xh[];
  __shared__ GemvLds lds;
  float *lut = lds.lut;
  float *part = lds.part;
  load_lut_lds(lut);
  if constexpr (XMODE == kXLds) {
    rms_to_lds(a.x, a.rms_w, a.K, a.rms_eps, xh, part);
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * kWavesPerWG + wave) * U;
  if (row0 >= a.M) {
    return;
  }
  const size_t pstride = static_cast<size_t>(a.K_pad >> 1);
  const size_t sstride = static_cast<size_t>(a.K_pad >> 6);
  const uint8_t *prow[U];
  const uint16_t *srow[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int r = min(row0 + u, a.M - 1);
    prow[u] = a.packed + r * pstride;
    srow[u] = a.scale + r * sstride;
  }
  float acc[U] = {};
  if constexpr (XMODE == kXGlobalFast) {
    rows_dot<U>(prow, srow, a.x, a.K_pad, lut, lane, acc);
  } else if constexpr (XMODE == kXGlobalGuarded) {
    rows_dot_guarded<U>(prow, srow, a.x, a.K, a.K_pad, lut, lane, acc);
  } else {
    rows_dot_guarded<U>(prow, srow, static_cast<const uint16_t *>(xh), a.K, a.K_pad, lut, lane,
                        acc);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float s = wave_sum(acc[u]);
    const int r = row0 + u;
    if (lane == u && r < a.M) {
      float v = s;
      if (a.add != nullptr) {
        v += bf16_to_f32(a.add[r]);
      }
      a.y[r] = f32_to_bf16(v);
    }
  }
}

// ---- fused q/k/v -------------------------------------------------------------
struct QkvArgs {
  const uint8_t *packed[3];
  const uint16_t *scale[3];
  uint16_t *y[3];
  const uint16_t *bias[3];
  int M[3];
  int blocks[3];  // workgroups given to each matrix
  const uint16_t *x;
  const uint16_t *rms_w;
  int K, K_pad;
  float rms_eps;
};

template <int U, int XMODE>
__global__ __launch_bounds__(kBlock) void gemv_qkv_rows(const QkvArgs a) {
  extern __shared__ uint16_t xh[];
  __shared__ GemvLds lds;
  float *lut = lds.lut;
  float *part = lds.part;
  load_lut_lds(lut);
  if constexpr (XMODE == kXLds) {
    rms_to_lds(a.x, a.rms_w, a.K, a.rms_eps, xh, part);
  }
  int b = blockIdx.x;
  int which = 0;
  if (b >= a.blocks[0]) {
    b -= a.blocks[0];
    which = 1;
    if (b >= a.blocks[1]) {
      b -= a.blocks[1];
      which = 2;
    }
  }
  const int M = a.M[which];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int row0 = (b * kWavesPerWG + wave) * U;
  if (row0 >= M) {
    return;
  }
  const size_t pstride = static_cast<size_t>(a.K_pad >> 1);
  const size_t sstride = static_cast<size_t>(a.K_pad >> 6);
  const uint8_t *prow[U];
  const uint16_t *srow[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int r = min(row0 + u, M - 1);
    prow[u] = a.packed[which] + r * pstride;
    srow[u] = a.scale[which] + r * sstride;
  }
  float acc[U] = {};
  if constexpr (XMODE == kXGlobalFast) {
    rows_dot<U>(prow, srow, a.x, a.K_pad, lut, lane, acc);
  } else if constexpr (XMODE == kXGlobalGuarded) {
    rows_dot_guarded<U>(prow, srow, a.x, a.K, a.K_pad, lut, lane, acc);
  } else {
    rows_dot_guarded<U>(prow, srow, static_cast<const uint16_t *>(xh), a.K, a.K_pad, lut, lane,
                        acc);
  }
  const uint16_t *bias = a.bias[which];
  uint16_t *y = a.y[which];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float s = wave_sum(acc[u]);
    const int r = row0 + u;
    if (lane == u && r < M) {
      float v = s;
      if (bias != nullptr) {
        v += bf16_to_f32(bias[r]);
      }
      y[r] = f32_to_bf16(v);
    }
  }
}

// ---- fused SwiGLU ------------------------------------------------------------
__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }

struct SwigluArgs {
  const uint8_t *gp;
  const uint16_t *gs;
  const uint8_t *up;
  const uint16_t *us;
  const uint16_t *x;
  uint16_t *y;
  const uint16_t *rms_w;
  int M, K, K_pad;
  float rms_eps;
};

// U gate rows and the matching U up rows per wavefront: 2U weight streams
// sharing one x.
template <int U, int XMODE>
__global__ __launch_bounds__(kBlock) void gemv_swiglu_rows(const SwigluArgs a) {
  extern __shared__ uint16_t xh[];
  __shared__ GemvLds lds;
  float *lut = lds.lut;
  float *part = lds.part;
  load_lut_lds(lut);
  if constexpr (XMODE == kXLds) {
    rms_to_lds(a.x, a.rms_w, a.K, a.rms_eps, xh, part);
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * kWavesPerWG + wave) * U;
  if (row0 >= a.M) {
    return;
  }
  const size_t pstride = static_cast<size_t>(a.K_pad >> 1);
  const size_t sstride = static_cast<size_t>(a.K_pad >> 6);
  const uint8_t *prow[2 * U];
  const uint16_t *srow[2 * U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int r = min(row0 + u, a.M - 1);
    prow[u] = a.gp + r * pstride;
    srow[u] = a.gs + r * sstride;
    prow[U + u] = a.up + r * pstride;
    srow[U + u] = a.us + r * sstride;
  }
  float acc[2 * U] = {};
  if constexpr (XMODE == kXGlobalFast) {
    rows_dot<2 * U>(prow, srow, a.x, a.K_pad, lut, lane, acc);
  } else if constexpr (XMODE == kXGlobalGuarded) {
    rows_dot_guarded<2 * U>(prow, srow, a.x, a.K, a.K_pad, lut, lane, acc);
  } else {
    rows_dot_guarded<2 * U>(prow, srow, static_cast<const uint16_t *>(xh), a.K, a.K_pad, lut,
                            lane, acc);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float g = wave_sum(acc[u]);
    const float v = wave_sum(acc[U + u]);
    const int r = row0 + u;
    if (lane == u && r < a.M) {
      a.y[r] = f32_to_bf16(silu(g) * v);
    }
  }
}

// ---- RMSNorm -----------------------------------------------------------------
constexpr int kRmsBlock = 1024;

__global__ __launch_bounds__(kRmsBlock) void rms_vec(const uint16_t *__restrict__ x,
                                                     const uint16_t *__restrict__ w,
                                                     uint16_t *__restrict__ y, int n, float eps) {
  __shared__ float part[kRmsBlock / kWave];
  float a = 0.f;
  for (int i = threadIdx.x; i < n; i += kRmsBlock) {
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
  for (int i = threadIdx.x; i < n; i += kRmsBlock) {
    y[i] = f32_to_bf16((bf16_to_f32(w[i]) * bf16_to_f32(x[i])) * inv);
  }
}

// ---- codec twins -------------------------------------------------------------
// One thread per packed dword (8 weights).  out is [M, K] fp32.
__global__ __launch_bounds__(256) void dequant_f32(const uint8_t *__restrict__ packed,
                                                   const uint16_t *__restrict__ scale,
                                                   float *__restrict__ out, int M, int K,
                                                   int K_pad) {
  __shared__ float lut[16];
  load_lut_lds(lut);
  const int dpr = K_pad >> 3;  // dwords per row
  const size_t total = static_cast<size_t>(M) * dpr;
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * 256) {
    const int r = static_cast<int>(i / dpr);
    const int d = static_cast<int>(i - static_cast<size_t>(r) * dpr);
    const uint32_t w = reinterpret_cast<const uint32_t *>(packed)[i];
    const float s = f16_to_f32(scale[static_cast<size_t>(r) * (K_pad >> 6) + (d >> 3)]);
    float *o = out + static_cast<size_t>(r) * K + (d << 3);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((d << 3) + j < K) {
        o[j] = lut[(w >> (4 * j)) & 0xFu] * s;
      }
    }
  }
}

// One workgroup per requested row; out is bf16 [n, K].
__global__ __launch_bounds__(256) void embed_rows(const uint8_t *__restrict__ packed,
                                                  const uint16_t *__restrict__ scale,
                                                  const int64_t *__restrict__ ids,
                                                  uint16_t *__restrict__ out, int M, int K,
                                                  int K_pad) {
  __shared__ float lut[16];
  load_lut_lds(lut);
  int64_t id = ids[blockIdx.x];
  if (id < 0 || id >= M) {
    // Out-of-range id: write zeros rather than read outside the table.
    for (int k = threadIdx.x; k < K; k += 256) {
      out[static_cast<size_t>(blockIdx.x) * K + k] = 0;
    }
    return;
  }
  const uint32_t *prow =
      reinterpret_cast<const uint32_t *>(packed + static_cast<size_t>(id) * (K_pad >> 1));
  const uint16_t *srow = scale + static_cast<size_t>(id) * (K_pad >> 6);
  uint16_t *o = out + static_cast<size_t>(blockIdx.x) * K;
  for (int d = threadIdx.x; d < (K_pad >> 3); d += 256) {
    const uint32_t w = prow[d];
    const float s = f16_to_f32(srow[d >> 3]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = (d << 3) + j;
      if (k < K) {
        o[k] = f32_to_bf16(lut[(w >> (4 * j)) & 0xFu] * s);
      }
    }
  }
}

// One wavefront per group of 64 weights: lane i owns column 64g + i.
// Steps are those of the CPU encoder (internal/nf4/nf4.go:129-185): absmax,
// binary16 scale, divide by the widened scale, clip, nearest level by squared
// distance in fp32 with the first minimum winning.
__global__ __launch_bounds__(256) void quantize_groups(const float *__restrict__ src,
                                                       uint8_t *__restrict__ packed,
                                                       uint16_t *__restrict__ scale,
                                                       int32_t *status, int M, int K, int K_pad) {
  const int lane = threadIdx.x & (kWave - 1);
  const int ng = K_pad >> 6;
  const size_t groups = static_cast<size_t>(M) * ng;
  const size_t wave_id = static_cast<size_t>(blockIdx.x) * (256 / kWave) + (threadIdx.x >> 6);
  const size_t n_waves = static_cast<size_t>(gridDim.x) * (256 / kWave);
  for (size_t gi = wave_id; gi < groups; gi += n_waves) {
    const int r = static_cast<int>(gi / ng);
    const int g = static_cast<int>(gi - static_cast<size_t>(r) * ng);
    const int c = (g << 6) + lane;
    const float v = c < K ? src[static_cast<size_t>(r) * K + c] : 0.f;
    const bool finite = (f32_to_bits(v) & 0x7F800000u) != 0x7F800000u;
    if (__any(!finite)) {
      if (lane == 0 && status != nullptr) {
        atomicOr(status, 1);
      }
      continue;
    }
    float s32 = group_max<64>(fabsf(v));
    if (s32 == 0.f) {
      s32 = 1.f;
    }
    uint16_t s16 = f32_to_f16_rne(s32);
    float s = f16_to_f32(s16);
    const bool bad = ((f32_to_bits(s) & 0x7F800000u) == 0x7F800000u) || !(s > 0.f);
    if (bad) {
      s32 = s32 > 65504.f ? 65504.f : 1.f;
      s16 = f32_to_f16_rne(s32);
      s = f16_to_f32(s16);
    }
    float u = v / s;
    u = u > 1.f ? 1.f : (u < -1.f ? -1.f : u);
    uint32_t best_j = 0;
    float d = u - bits_to_f32(kLutBits[0]);
    float best = d * d;
#pragma unroll
    for (uint32_t j = 1; j < 16; ++j) {
      d = u - bits_to_f32(kLutBits[j]);
      const float d2 = d * d;
      if (d2 < best) {
        best = d2;
        best_j = j;
      }
    }
    const uint32_t hi = static_cast<uint32_t>(__shfl_down(static_cast<int>(best_j), 1, kWave));
    if ((lane & 1) == 0) {
      packed[static_cast<size_t>(r) * (K_pad >> 1) + (g << 5) + (lane >> 1)] =
          static_cast<uint8_t>((hi << 4) | best_j);
    }
    if (lane == 0) {
      scale[gi] = s16;
    }
  }
}

int pick_rows(int M) {
  const char *e = std::getenv("CHR_NF4_GEMV_NR");
  if (e != nullptr && e[0] != '\0') {
    const int v = std::atoi(e);
    if (v == 1 || v == 2 || v == 4 || v == 8) {
      return v;
    }
  }
  if (M >= 8192) {
    return 4;
  }
  if (M >= 2048) {
    return 2;
  }
  return 1;
}

int desc_rc(const chr_nf4_dev_t *w) {
  if (w->M < 1 || w->K < 1 || w->packed == nullptr || w->scale == nullptr) {
    return -3;
  }
  if (!k_pad_ok(w->K, w->K_pad)) {
    return -4;
  }
  return 0;
}

constexpr size_t kMaxDynLds = 160 * 1024 - 1024;

template <typename Kern>
int prep_lds(Kern kern, size_t dyn) {
  if (dyn > kMaxDynLds) {
    return -6;
  }
  if (dyn > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(dyn)) != hipSuccess) {
      return -6;
    }
  }
  return 0;
}

template <int U>
int launch_gemv(const GemvArgs &a, hipStream_t st) {
  const dim3 grid((a.M + kWavesPerWG * U - 1) / (kWavesPerWG * U));
  const dim3 block(kBlock);
  if (a.rms_w != nullptr) {
    const size_t dyn = static_cast<size_t>(a.K) * 2;
    if (prep_lds(gemv_rows<U, kXLds>, dyn) != 0) {
      return -6;
    }
    gemv_rows<U, kXLds><<<grid, block, dyn, st>>>(a);
  } else if (a.K == a.K_pad) {
    gemv_rows<U, kXGlobalFast><<<grid, block, 0, st>>>(a);
  } else {
    gemv_rows<U, kXGlobalGuarded><<<grid, block, 0, st>>>(a);
  }
  return launch_rc();
}

template <int U>
int launch_swiglu(const SwigluArgs &a, hipStream_t st) {
  const dim3 grid((a.M + kWavesPerWG * U - 1) / (kWavesPerWG * U));
  const dim3 block(kBlock);
  if (a.rms_w != nullptr) {
    const size_t dyn = static_cast<size_t>(a.K) * 2;
    if (prep_lds(gemv_swiglu_rows<U, kXLds>, dyn) != 0) {
      return -6;
    }
    gemv_swiglu_rows<U, kXLds><<<grid, block, dyn, st>>>(a);
  } else if (a.K == a.K_pad) {
    gemv_swiglu_rows<U, kXGlobalFast><<<grid, block, 0, st>>>(a);
  } else {
    gemv_swiglu_rows<U, kXGlobalGuarded><<<grid, block, 0, st>>>(a);
  }
  return launch_rc();
}

template <int U>
int launch_qkv(QkvArgs &a, hipStream_t st) {
  int total = 0;
  for (int i = 0; i < 3; ++i) {
    a.blocks[i] = (a.M[i] + kWavesPerWG * U - 1) / (kWavesPerWG * U);
    total += a.blocks[i];
  }
  const dim3 grid(total);
  const dim3 block(kBlock);
  if (a.rms_w != nullptr) {
    const size_t dyn = static_cast<size_t>(a.K) * 2;
    if (prep_lds(gemv_qkv_rows<U, kXLds>, dyn) != 0) {
      return -6;
    }
    gemv_qkv_rows<U, kXLds><<<grid, block, dyn, st>>>(a);
  } else if (a.K == a.K_pad) {
    gemv_qkv_rows<U, kXGlobalFast><<<grid, block, 0, st>>>(a);
  } else {
    gemv_qkv_rows<U, kXGlobalGuarded><<<grid, block, 0, st>>>(a);
  }
  return launch_rc();
}

}  // namespace

// Shared with the GEMM entry points, which route N == 1 here.
int gemv_entry(const chr_nf4_dev_t *w, const void *x, void *y, void *stream, const void *add,
               const void *rms_w, float rms_eps) {
  if (w == nullptr || x == nullptr || y == nullptr) {
    return -1;
  }
  if (const int rc = desc_rc(w)) {
    return rc;
  }
  if (!aligned16(w->packed) || !aligned16(x) || !aligned2(w->scale)) {
    return -5;
  }
  GemvArgs a{};
  a.packed = w->packed;
  a.scale = w->scale;
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.add = static_cast<const uint16_t *>(add);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.M = w->M;
  a.K = w->K;
  a.K_pad = w->K_pad;
  a.rms_eps = rms_eps;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (pick_rows(w->M)) {
    case 8:
      return launch_gemv<8>(a, st);
    case 4:
      return launch_gemv<4>(a, st);
    case 2:
      return launch_gemv<2>(a, st);
    default:
      return launch_gemv<1>(a, st);
  }
}

int gemv_rows_per_wg(int M) { return kWavesPerWG * pick_rows(M); }

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
  QkvArgs a{};
  const chr_nf4_dev_t *m[3] = {q, k, v};
  void *ys[3] = {yq, yk, yv};
  const void *bs[3] = {bq, bk, bv};
  for (int i = 0; i < 3; ++i) {
    a.packed[i] = m[i]->packed;
    a.scale[i] = m[i]->scale;
    a.y[i] = static_cast<uint16_t *>(ys[i]);
    a.bias[i] = static_cast<const uint16_t *>(bs[i]);
    a.M[i] = m[i]->M;
  }
  a.x = static_cast<const uint16_t *>(x);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.K = q->K;
  a.K_pad = q->K_pad;
  a.rms_eps = rms_eps;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (pick_rows(q->M + k->M + v->M)) {
    case 8:
      return launch_qkv<8>(a, st);
    case 4:
      return launch_qkv<4>(a, st);
    case 2:
      return launch_qkv<2>(a, st);
    default:
      return launch_qkv<1>(a, st);
  }
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
  SwigluArgs a{};
  a.gp = gate->packed;
  a.gs = gate->scale;
  a.up = up->packed;
  a.us = up->scale;
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.rms_w = static_cast<const uint16_t *>(rms_w);
  a.M = gate->M;
  a.K = gate->K;
  a.K_pad = gate->K_pad;
  a.rms_eps = rms_eps;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Two weight streams per output row: half the rows per wavefront of the
  // plain GEMV keeps the same number of loads in flight.
  const int u = pick_rows(gate->M);
  if (u >= 4) {
    return launch_swiglu<2>(a, st);
  }
  if (u == 2) {
    return launch_swiglu<1>(a, st);
  }
  return launch_swiglu<1>(a, st);
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

extern "C" int chr_nf4_dequant(const chr_nf4_dev_t *w, float *out, void *stream) {
  if (w == nullptr || out == nullptr) {
    return -1;
  }
  if (const int rc = desc_rc(w)) {
    return rc;
  }
  if ((reinterpret_cast<uintptr_t>(w->packed) & 3u) != 0 || !aligned2(w->scale)) {
    return -5;
  }
  const size_t total = static_cast<size_t>(w->M) * (w->K_pad >> 3);
  const unsigned blocks = static_cast<unsigned>(std::min<size_t>((total + 255) / 256, 65536));
  dequant_f32<<<dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      w->packed, w->scale, out, w->M, w->K, w->K_pad);
  return launch_rc();
}

extern "C" int chr_nf4_embed_rows(const chr_nf4_dev_t *table, const void *ids, int32_t n,
                                  void *out, void *stream) {
  if (table == nullptr || ids == nullptr || out == nullptr) {
    return -1;
  }
  if (n < 1) {
    return -2;
  }
  if (const int rc = desc_rc(table)) {
    return rc;
  }
  if ((reinterpret_cast<uintptr_t>(table->packed) & 3u) != 0 || !aligned2(table->scale)) {
    return -5;
  }
  embed_rows<<<dim3(static_cast<unsigned>(n)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      table->packed, table->scale, static_cast<const int64_t *>(ids),
      static_cast<uint16_t *>(out), table->M, table->K, table->K_pad);
  return launch_rc();
}

extern "C" int chr_nf4_quantize(const float *src, const chr_nf4_dev_t *dst, int32_t *status,
                                void *stream) {
  if (src == nullptr || dst == nullptr) {
    return -1;
  }
  if (const int rc = desc_rc(dst)) {
    return rc;
  }
  const size_t groups = static_cast<size_t>(dst->M) * (dst->K_pad >> 6);
  const unsigned blocks = static_cast<unsigned>(std::min<size_t>((groups + 3) / 4, 1u << 20));
  quantize_groups<<<dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      src, const_cast<uint8_t *>(dst->packed), const_cast<uint16_t *>(dst->scale), status, dst->M,
      dst->K, dst->K_pad);
  return launch_rc();
}

extern "C" int chr_nf4_abi_version(void) { return 1; }

// Codec twins of the CPU NF4 codec on gfx950: full-matrix dequant to fp32,
// embedding-row gather to bf16, and the quantiser that makes synthetic weights.
// Device counterparts of internal/nf4/nf4.go:46-121,129-185 and
// gpu/host/embedding.py:74-107; each is bit-exact against the CPU codec.

#include "nf4_common.h"

#include <algorithm>

namespace chr {
namespace {

__device__ __forceinline__ void load_lut_lds(float *lut) {
  if (threadIdx.x < 16) {
    lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  __syncthreads();
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

int desc_rc(const chr_nf4_dev_t *w) {
  if (w->M < 1 || w->K < 1 || w->packed == nullptr || w->scale == nullptr) {
    return -3;
  }
  if (!k_pad_ok(w->K, w->K_pad)) {
    return -4;
  }
  return 0;
}

}  // namespace
}  // namespace chr

using namespace chr;

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

// Device-side bookkeeping of the resident decode step, so that a greedy step
// needs no host read and only one small launch at each end:
//   chr_dv2_mark_written   valid_len = position + 1   (gpu/decodev2/kv.py:118-120)
//   chr_dv2_argmax_commit  next = argmax(logits), then token = next,
//                          position += 1, finished |= (next == eos)
//                          (gpu/decodev2/step.py:182, gpu/decodev2/state.py:98-103)
// The argmax runs on the bf16 logits as stored and the lowest index wins a tie,
// which is what the CPU oracle's argmax does.

#include "nf4_common.h"

namespace chr {

int gemv_attn_entry(const chr_nf4_dev_t *w, const float *state, int n_q, int hd, int n_parts,
                    void *y, const void *add, void *stream, float *sq_out);

namespace {

constexpr int kBeginBlock = 1024;

// First launch of a fused decode step, one workgroup:
//   valid_len = position + 1
//   x   = bf16( LUT[code] * f32(scale) ) for row *token of the packed embedding
//   h   = RMSNorm(x, norm_w, eps) rounded to bf16, when norm_w is given
// i.e. GraphSafeKV.mark_written + the embedding gather (+ the first RMSNorm).
__global__ __launch_bounds__(kBeginBlock) void begin_step(
    const uint8_t *__restrict__ packed, const uint16_t *__restrict__ scale, int M, int K, int K_pad,
    const int64_t *__restrict__ token, const int64_t *__restrict__ position,
    int32_t *__restrict__ valid_len, uint16_t *__restrict__ x, const uint16_t *__restrict__ norm_w,
    float eps, uint16_t *__restrict__ h, float *__restrict__ sq_out, int sq_parts) {
  __shared__ float lut[16];
  __shared__ float part[kBeginBlock / kWave];
  if (threadIdx.x < 16) {
    lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  if (threadIdx.x == 0) {
    *valid_len = static_cast<int32_t>(*position) + 1;
  }
  __syncthreads();
  const int64_t id = *token;
  const bool ok = id >= 0 && id < M;  // an id outside the table decodes to zeros
  const uint32_t *prow =
      reinterpret_cast<const uint32_t *>(packed + static_cast<size_t>(ok ? id : 0) * (K_pad >> 1));
  const uint16_t *srow = scale + static_cast<size_t>(ok ? id : 0) * (K_pad >> 6);
  float sq = 0.f;
  for (int d = threadIdx.x; d < (K_pad >> 3); d += kBeginBlock) {
    const uint32_t w = ok ? prow[d] : 0x77777777u;
    const float s = ok ? f16_to_f32(srow[d >> 3]) : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = (d << 3) + j;
      if (k < K) {
        const uint16_t b = f32_to_bf16(lut[(w >> (4 * j)) & 0xFu] * s);
        x[k] = b;
        const float v = bf16_to_f32(b);
        sq = fmaf(v, v, sq);
      }
    }
  }
  sq = wave_sum(sq);
  if ((threadIdx.x & (kWave - 1)) == 0) {
    part[threadIdx.x >> 6] = sq;
  }
  if (norm_w == nullptr && sq_out == nullptr) {
    return;
  }
  __syncthreads();  // also orders this workgroup's x stores before the reads below
  if (sq_out != nullptr) {
    // the sum of squares of x in the form the GEMVs hand it on: the wavefronts' sums as the
    // first parts, zeros behind them
    for (int i = threadIdx.x; i < sq_parts; i += kBeginBlock) {
      sq_out[i] = i < kBeginBlock / kWave ? part[i] : 0.f;
    }
  }
  if (norm_w == nullptr) {
    return;
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kBeginBlock / kWave; ++i) {
    sum += part[i];
  }
  const float inv = rsqrtf(sum / static_cast<float>(K) + eps);
  for (int d = threadIdx.x; d < (K_pad >> 3); d += kBeginBlock) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = (d << 3) + j;
      if (k < K) {
        // each thread re-reads only what it stored itself
        h[k] = f32_to_bf16((bf16_to_f32(norm_w[k]) * bf16_to_f32(x[k])) * inv);
      }
    }
  }
}

__global__ void mark_written(const int64_t *__restrict__ position, int32_t *__restrict__ valid_len) {
  if (threadIdx.x == 0) {
    *valid_len = static_cast<int32_t>(*position) + 1;
  }
}

constexpr int kArgmaxBlock = 1024;

// Total order on (value, index): larger value first, then smaller index.  NaN
// compares as larger than everything, so a NaN logit is surfaced, not hidden.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  const bool vn = v != v, bn = bv != bv;
  if (vn != bn) {
    return vn;
  }
  if (vn && bn) {
    return i < bi;
  }
  return v > bv || (v == bv && i < bi);
}

__global__ __launch_bounds__(kArgmaxBlock) void argmax_commit(
    const uint16_t *__restrict__ logits, int n, int64_t *__restrict__ next_token,
    int64_t *__restrict__ token, int64_t *__restrict__ position, uint8_t *__restrict__ finished,
    const int64_t *__restrict__ eos_id, int commit) {
  __shared__ float sv[kArgmaxBlock / kWave];
  __shared__ int si[kArgmaxBlock / kWave];
  float bv = -__builtin_inff();
  int bi = 0x7FFFFFFF;
  // Eight logits per 16-byte load when the buffer allows it; indices rise within
  // a thread, so "strictly better" keeps the lowest index of equal values.
  const bool vec = (reinterpret_cast<uintptr_t>(logits) & 15u) == 0;
  const int n8 = vec ? n >> 3 : 0;
  // kBatch loads are in flight together: one workgroup walks the whole vocabulary, so the
  // loop is a chain of memory round trips and their number is what it costs
  constexpr int kBatch = 8;
  for (int c0 = threadIdx.x; c0 < n8; c0 += kArgmaxBlock * kBatch) {
    uint4 raw[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int c = c0 + b * kArgmaxBlock;
      raw[b] = reinterpret_cast<const uint4 *>(logits)[c < n8 ? c : c0];
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int c = c0 + b * kArgmaxBlock;
      if (c < n8) {
        const uint32_t w[4] = {raw[b].x, raw[b].y, raw[b].z, raw[b].w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float v = (j & 1) ? bf16_hi(w[j >> 1]) : bf16_lo(w[j >> 1]);
          const int i = (c << 3) + j;
          if (better(v, i, bv, bi)) {
            bv = v;
            bi = i;
          }
        }
      }
    }
  }
  for (int i = (n8 << 3) + threadIdx.x; i < n; i += kArgmaxBlock) {
    const float v = bf16_to_f32(logits[i]);
    if (better(v, i, bv, bi)) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    sv[threadIdx.x >> 6] = bv;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxBlock / kWave; ++w) {
      if (better(sv[w], si[w], bv, bi)) {
        bv = sv[w];
        bi = si[w];
      }
    }
    const int64_t nt = bi;
    *next_token = nt;
    if (commit) {
      *token = nt;
      *position += 1;
      if (nt == *eos_id) {
        *finished |= 1;
      }
    }
  }
}

// The same argmax over a large vocabulary as two launches: kArgmaxParts workgroups each
// leave the best (value, index) of a contiguous slice, a small one picks among them and
// commits.  One workgroup walking 150 K logits takes ~32 us; this pair ~8 us.
constexpr int kArgmaxParts = 128;
constexpr int kArgmaxPartBlock = 256;

struct Candidate {
  float v;
  int i;
};

__global__ __launch_bounds__(kArgmaxPartBlock) void argmax_parts(const uint16_t *__restrict__ logits,
                                                                 int n, int slice,
                                                                 Candidate *__restrict__ ws) {
  __shared__ float sv[kArgmaxPartBlock / kWave];
  __shared__ int si[kArgmaxPartBlock / kWave];
  const int lo = static_cast<int>(blockIdx.x) * slice;  // slice is a multiple of 8
  const int hi = min(n, lo + slice);
  float bv = -__builtin_inff();
  int bi = 0x7FFFFFFF;
  const bool vec = (reinterpret_cast<uintptr_t>(logits) & 15u) == 0;
  const int c_lo = lo >> 3;
  const int c_hi = vec ? hi >> 3 : c_lo;  // whole 8-logit vectors of the slice
  for (int c = c_lo + threadIdx.x; c < c_hi; c += kArgmaxPartBlock) {
    const uint4 raw = reinterpret_cast<const uint4 *>(logits)[c];
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (j & 1) ? bf16_hi(w[j >> 1]) : bf16_lo(w[j >> 1]);
      const int i = (c << 3) + j;
      if (better(v, i, bv, bi)) {
        bv = v;
        bi = i;
      }
    }
  }
  for (int i = (c_hi << 3) + threadIdx.x; i < hi; i += kArgmaxPartBlock) {
    const float v = bf16_to_f32(logits[i]);
    if (better(v, i, bv, bi)) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    sv[threadIdx.x >> 6] = bv;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxPartBlock / kWave; ++w) {
      if (better(sv[w], si[w], bv, bi)) {
        bv = sv[w];
        bi = si[w];
      }
    }
    ws[blockIdx.x].v = bv;  // an empty slice leaves (-inf, INT_MAX): never the winner
    ws[blockIdx.x].i = bi;
  }
}

__global__ __launch_bounds__(kArgmaxParts) void argmax_final(
    const Candidate *__restrict__ ws, int64_t *__restrict__ next_token, int64_t *__restrict__ token,
    int64_t *__restrict__ position, uint8_t *__restrict__ finished,
    const int64_t *__restrict__ eos_id, int commit) {
  __shared__ float sv[kArgmaxParts / kWave];
  __shared__ int si[kArgmaxParts / kWave];
  float bv = ws[threadIdx.x].v;
  int bi = ws[threadIdx.x].i;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    sv[threadIdx.x >> 6] = bv;
    si[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxParts / kWave; ++w) {
      if (better(sv[w], si[w], bv, bi)) {
        bv = sv[w];
        bi = si[w];
      }
    }
    const int64_t nt = bi;
    *next_token = nt;
    if (commit) {
      *token = nt;
      *position += 1;
      if (nt == *eos_id) {
        *finished |= 1;
      }
    }
  }
}

}  // namespace
}  // namespace chr

using namespace chr;

namespace chr {
namespace {
int begin_step_entry(const chr_nf4_dev_t *table, const void *token, const void *position,
                     void *valid_len, void *x, const void *norm_w, float eps, void *h, void *stream,
                     float *sq_out) {
  if (table == nullptr || token == nullptr || position == nullptr || valid_len == nullptr ||
      x == nullptr || (norm_w != nullptr && h == nullptr)) {
    return -1;
  }
  if (table->M < 1 || table->K < 1 || table->packed == nullptr || table->scale == nullptr) {
    return -3;
  }
  if (!k_pad_ok(table->K, table->K_pad)) {
    return -4;
  }
  if ((reinterpret_cast<uintptr_t>(table->packed) & 3u) != 0 || !aligned2(table->scale)) {
    return -5;
  }
  begin_step<<<dim3(1), dim3(kBeginBlock), 0, static_cast<hipStream_t>(stream)>>>(
      table->packed, table->scale, table->M, table->K, table->K_pad,
      static_cast<const int64_t *>(token), static_cast<const int64_t *>(position),
      static_cast<int32_t *>(valid_len), static_cast<uint16_t *>(x),
      static_cast<const uint16_t *>(norm_w), eps, static_cast<uint16_t *>(h), sq_out, kSumsqParts);
  return launch_rc();
}
}  // namespace
}  // namespace chr

extern "C" int chr_dv2_begin_step(const chr_nf4_dev_t *table, const void *token,
                                  const void *position, void *valid_len, void *x,
                                  const void *norm_w, float eps, void *h, void *stream) {
  return begin_step_entry(table, token, position, valid_len, x, norm_w, eps, h, stream, nullptr);
}

extern "C" int chr_dv2_begin_step_sumsq(const chr_nf4_dev_t *table, const void *token,
                                        const void *position, void *valid_len, void *x,
                                        void *stream, float *sumsq_out) {
  if (sumsq_out == nullptr || (reinterpret_cast<uintptr_t>(sumsq_out) & 3u) != 0) {
    return sumsq_out == nullptr ? -1 : -5;
  }
  return begin_step_entry(table, token, position, valid_len, x, nullptr, 0.f, nullptr, stream,
                          sumsq_out);
}

extern "C" int chr_dv2_gemv_attn(const chr_nf4_dev_t *w, const float *state, int32_t n_q,
                                 int32_t hd, int32_t n_parts, void *y, const void *add,
                                 void *stream) {
  return gemv_attn_entry(w, state, n_q, hd, n_parts, y, add, stream, nullptr);
}

extern "C" int chr_dv2_gemv_attn_sumsq(const chr_nf4_dev_t *w, const float *state, int32_t n_q,
                                       int32_t hd, int32_t n_parts, void *y, const void *add,
                                       void *stream, float *sumsq_out) {
  return gemv_attn_entry(w, state, n_q, hd, n_parts, y, add, stream, sumsq_out);
}

extern "C" int chr_dv2_mark_written(const void *position, void *valid_len, void *stream) {
  if (position == nullptr || valid_len == nullptr) {
    return -1;
  }
  mark_written<<<dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const int64_t *>(position), static_cast<int32_t *>(valid_len));
  return launch_rc();
}

extern "C" int chr_dv2_argmax_commit(const void *logits, int32_t n, void *next_token, void *token,
                                     void *position, void *finished, const void *eos_id,
                                     int32_t commit, void *stream) {
  if (logits == nullptr || next_token == nullptr) {
    return -1;
  }
  if (commit != 0 && (token == nullptr || position == nullptr || finished == nullptr ||
                      eos_id == nullptr)) {
    return -1;
  }
  if (n < 1) {
    return -3;
  }
  argmax_commit<<<dim3(1), dim3(kArgmaxBlock), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint16_t *>(logits), n, static_cast<int64_t *>(next_token),
      static_cast<int64_t *>(token), static_cast<int64_t *>(position),
      static_cast<uint8_t *>(finished), static_cast<const int64_t *>(eos_id), commit);
  return launch_rc();
}

extern "C" int64_t chr_dv2_argmax_ws_bytes(void) {
  return static_cast<int64_t>(kArgmaxParts) * static_cast<int64_t>(sizeof(Candidate));
}

extern "C" int chr_dv2_argmax_commit_ws(const void *logits, int32_t n, void *next_token,
                                        void *token, void *position, void *finished,
                                        const void *eos_id, int32_t commit, void *ws,
                                        int64_t ws_bytes, void *stream) {
  constexpr int kSmall = 16384;  // below this one workgroup is as quick as two launches
  if (ws == nullptr || ws_bytes < chr_dv2_argmax_ws_bytes() || n < kSmall ||
      (reinterpret_cast<uintptr_t>(ws) & 7u) != 0) {
    return chr_dv2_argmax_commit(logits, n, next_token, token, position, finished, eos_id, commit,
                                 stream);
  }
  if (logits == nullptr || next_token == nullptr) {
    return -1;
  }
  if (commit != 0 && (token == nullptr || position == nullptr || finished == nullptr ||
                      eos_id == nullptr)) {
    return -1;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int slice = ((n + kArgmaxParts - 1) / kArgmaxParts + 7) & ~7;
  argmax_parts<<<dim3(kArgmaxParts), dim3(kArgmaxPartBlock), 0, st>>>(
      static_cast<const uint16_t *>(logits), n, slice, static_cast<Candidate *>(ws));
  argmax_final<<<dim3(1), dim3(kArgmaxParts), 0, st>>>(
      static_cast<const Candidate *>(ws), static_cast<int64_t *>(next_token),
      static_cast<int64_t *>(token), static_cast<int64_t *>(position),
      static_cast<uint8_t *>(finished), static_cast<const int64_t *>(eos_id), commit);
  return launch_rc();
}

// N=1 NF4 GEMV family for gfx950 (MI355X): plain / residual-add, fused q-k-v,
// fused SwiGLU, and RMSNorm.  Replaces the entry points of
// gpu/nf4/nf4_gemv.cu:790-924, 996-1011.
//
// Two kernels, chosen per launch (pick_family).
//
// Staged (gemv_staged): one workgroup of 16 wavefronts per compute unit.  x is copied to
// LDS once per workgroup (RMS-normalised, zero-padded or merged from attention states on
// the way if asked).  Packed bytes are looked up two codes at a time in a 256-entry table
// of bf16 level pairs of which every lane owns a copy (conflict-free for any codes), and
// meet the matching bf16 pair of x in one v_dot2c_f32_bf16.  Lane l of half step t reads
// the 8 packed bytes 8*(64t + l) of a row; requests run one two-step item ahead of the
// arithmetic through two register buffers.  Taken for a fused RMSNorm, a ragged K, the
// attention merge, and every launch of 16M codes or more.
//
// Plain (gemv_stream): four wavefronts per workgroup; every wavefront owns R weight rows
// and walks the whole K axis of each.  Lane l reads the 16-byte chunk l + 64*j of a row
// (the K remainder as 8-byte half chunks, so K = 5120 costs 2 + 1 steps), x comes straight
// from global memory, and the 16 fp32 levels sit at LDS address 0: 16 distinct addresses
// in 16 distinct banks, a lookup address is one byte-select AND.  Taken for small launches,
// where the staged kernel's set-up costs more than its inner loop returns.
//
// Numerics.  Plain: weight = fp32 LUT * fp32(scale) never rounded below fp32, x widened
// bf16->fp32 (gpu/nf4/nf4_gemv.cu:70-101, 217-245).  Staged and ring kernels, by the form of
// the levels (CHR_NF4_GEMV_TERMS): 3, the default: levels rounded to binary16 (2^-12 relative)
// against x staged as binary16, every 16 consecutive activations times a power of two of
// their own, which holds every bf16 element within 2^-29 of the largest of its 16 exactly;
// 2: levels as two bf16 terms (below 2^-17), 8-byte lookups;
// 1: levels rounded to bf16 (2^-9), the precision class of the reference's tensor-core path
// (gpu/nf4/nf4_gemm.cu:322).  In all three the products are exact and the fp16 scale is
// applied in fp32 to each 16-weight partial.  Both families: fp32 accumulation, residual /
// bias added in fp32, one bf16 rounding at the store.

#include "nf4_common.h"
#include "nf4_gemv_ring_regs.h"

#include <algorithm>
#include <cstdlib>

namespace chr {
namespace {

constexpr int kMaxWaves = 16;  // wavefronts per workgroup, upper bound
constexpr int kThreads = 256;          // workgroup of the plain kernel, fixed
constexpr int kStagedThreads = 1024;  // workgroup of the kernel that stages x in LDS, fixed

// Static LDS of the GEMV kernels.  The codebook comes first so that its LDS
// address is 0 and a lookup address is just 4*code.
struct GemvLds {
  float lut[16];
  float part[kMaxWaves];
  float ksum[kMaxWaves][4];  // K-split: per-wavefront partial dot products of a row group
};

// The small statics of the kernels that stage x in LDS (their slot of kStagedSmallBytes).
struct StagedLds : GemvLds {};

__device__ __forceinline__ float fma8(const Levels8 &v, const float *xf, float acc) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    acc = fmaf(v.l[j], xf[j], acc);
  }
  return acc;
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
  // ring kernels: grid size, full passes of 16 * grid groups, and the groups left after them
  int ring_grid, ring_passes, ring_left;
  // Sum of squares handed from the launch that writes a vector to the launch that normalises
  // it: kSumsqParts floats, workgroup b of the writer leaving the sum over its rows' stored
  // bf16 values at [b] (zeros where no workgroup writes).  sq_out: this launch writes them for
  // its y; sq_in (with rms_w): this launch takes mean(x^2) from them instead of summing x.
  float *sq_out;
  const float *sq_in;
};

// Sum of a value over a workgroup of kStagedThreads threads, the same in every thread.
__device__ __forceinline__ float block_sum(float v, float *part) {
  v = wave_sum(v);
  const int waves = kStagedThreads >> 6;
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

// sq_out at the end of a launch (every wavefront of the workgroup calls it): the wavefronts' sums
// of squares meet in their own order, the workgroup stores its part, and zeros at the places
// that no workgroup of this grid writes.
__device__ __forceinline__ void store_sumsq_part(const StreamArgs &a, StagedLds &lds, float sq_acc,
                                                 int wave, int lane) {
  if (lane == 0) {
    lds.part[wave] = sq_acc;
  }
  __syncthreads();
  if (wave == 0 && lane == 0) {
    float s = 0.f;
    for (int w = 0; w < (kStagedThreads >> 6); ++w) {
      s += lds.part[w];
    }
    const int block = static_cast<int>(blockIdx.x);
    a.sq_out[block] = s;
    for (int b = block + a.ring_grid; b < kSumsqParts; b += a.ring_grid) {
      a.sq_out[b] = 0.f;
    }
  }
}

// ---- x as binary16 -------------------------------------------------------------------
// With levels kept as binary16 (11 significant bits against bf16's 8) the products need x as
// binary16 too.  A bf16 value has 8 significant bits, so it is a binary16 value exactly
// whenever its exponent fits.  The 16 activations one lane multiplies in one half step (two
// 16-byte pieces, staged by two neighbouring threads) are therefore multiplied by the power
// of two that puts the largest of them in [2^14, 2^15): every one within 2^-29 of that
// largest converts exactly, smaller ones land on binary16's subnormal grid (absolute error
// below 2^-39 of the largest: far under the fp32 accumulation's own rounding).  The inverse
// power is kept beside x as a float, one per pair of pieces, and multiplies the fp16 scale of
// the lane's 16 weights before it meets their sum.  A pair of zeros, or one that holds
// something not finite: power 0 (what is not finite stays so through the products).
typedef uint16_t U16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(U16x2, a),
                                                                __builtin_bit_cast(U16x2, b)));
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
}

// The power for the pair of pieces this thread and its neighbour (lane ^ 1) hold: the
// magnitude bits of a bf16 value order like its magnitude, so the largest of the 16 is an
// unsigned 16-bit maximum.  Every lane of the wavefront must be active (the neighbour's
// value is read across lanes); a thread without a piece passes zeros.
__device__ __forceinline__ int pair_power(const uint4 &piece) {
  const uint32_t mask = 0x7FFF7FFFu;
  uint32_t m = pk_max_u16(pk_max_u16(piece.x & mask, piece.y & mask), pk_max_u16(piece.z & mask, piece.w & mask));
  m = max(m & 0xFFFFu, m >> 16);
  m = max(m, dpp_u32<kDppQuadXor1>(m));
  if (m == 0u || m >= 0x7F80u) {
    return 0;
  }
  // exponent field -127: -113 for the largest bf16, 141 for a subnormal (read as exponent
  // -127; it ends up below 2^15 too)
  return 14 - (static_cast<int>(m >> 7) - 127);
}

// two bf16 values (one dword) -> the same two values times 2^power as a binary16 pair
__device__ __forceinline__ uint32_t bf16x2_to_f16x2(uint32_t pair, int power) {
  const float lo = __builtin_ldexpf(bf16_lo(pair), power);
  const float hi = __builtin_ldexpf(bf16_hi(pair), power);
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

__device__ __forceinline__ uint4 piece_to_f16(const uint4 &piece, int power) {
  return make_uint4(bf16x2_to_f16x2(piece.x, power), bf16x2_to_f16x2(piece.y, power),
                    bf16x2_to_f16x2(piece.z, power), bf16x2_to_f16x2(piece.w, power));
}

// ---- activations staged in LDS ------------------------------------------------------
// A "piece" is 8 consecutive activations (16 bytes of bf16).  The staged kernel walks a
// row in steps of 64 lanes x 8 packed bytes: lane l of step t holds the 16 codes of half
// chunk h = 64t + l and needs pieces 2h and 2h+1.  They are stored as [t][q][l], so one
// ds_read_b128 of the wavefront covers 64 consecutive pieces (no bank conflicts).
__host__ __device__ inline int x_half_steps(int K_pad) { return ((K_pad >> 4) + kWave - 1) >> 6; }

__host__ __device__ inline int x_pieces(int K_pad) { return x_half_steps(K_pad) * 128; }

__device__ __forceinline__ int x_slot(int piece) {
  const int h = piece >> 1, q = piece & 1;
  return ((h >> 6) << 7) + (q << 6) + (h & 63);
}

// Zero the slots of the last step that no piece of the row maps to.
__device__ __forceinline__ void zero_unused_slots(uint4 *xs, int K_pad) {
  const int n_half = K_pad >> 4;
  const int last = (x_half_steps(K_pad) - 1) << 7;
  for (int i = last + threadIdx.x; i < last + 128; i += kStagedThreads) {
    const int h = ((last >> 7) << 6) + (i & 63);
    if (h >= n_half) {
      xs[i] = make_uint4(0, 0, 0, 0);
    }
  }
}

// Fill the LDS copy: zero for k in [K, K_pad) and for unused slots.  With rms_w the
// value stored is bf16( (w*x) * rsqrt(mean(x^2)+eps) ), i.e. what a separate RMSNorm
// launch would have handed over (gpu/nf4/nf4_gemv.cu:264-289).  Used for a ragged K
// and for the fused RMSNorm.
// x piece i (8 consecutive dims of one head) merged from the per-part softmax states:
// x = sum_p e^{m_p - M} o_p / sum_p e^{m_p - M} l_p, rounded to bf16 as the attention
// launch itself would have stored it.  An empty part has m = -1e30, l = 0: weight zero.
template <int kBatch>  // parts whose states are fetched together (one memory round trip)
__device__ __forceinline__ uint4 merged_attn_piece(const StreamArgs &a, int i) {
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
    r[q] = f32x2_to_bf16x2(o[2 * q] * inv, o[2 * q + 1] * inv);
  }
  return make_uint4(r[0], r[1], r[2], r[3]);
}

constexpr int kXKeep = 4;  // 16-byte vectors of x a thread keeps between request and use

// Threads the 16-byte vectors of x are dealt over in the fast staging (vector i to thread
// i % deal, its round i / deal): the first eight wavefronts where x fits their kXKeep rounds,
// all sixteen beyond.  The wavefronts that hold no x write their share of the level table and
// wait at the barrier; with eight rather than sixteen (or the ten that 640 vectors would take
// at one each) asking for x, its requests queue behind fewer of the first weight requests:
// 5120x13824 10.35 -> 10.0 us, 13824x5120 9.35 -> 9.25 us, 14B decode +1% (256 and 384
// threads: no better).
constexpr int kXDeal = 512;
static_assert(kXDeal <= kStagedThreads && kXDeal % 128 == 0, "whole pairs of wavefront lanes");
__device__ __forceinline__ int x_deal(int nk) {
  return nk <= kXKeep * kXDeal ? kXDeal : kStagedThreads;
}

// The common case of staging: K a multiple of 8, aligned pointers, x short enough to sit in
// registers between its request and its use, no attention merge.
__device__ __forceinline__ bool stage_fast_ok(const StreamArgs &a) {
  return a.attn_state == nullptr && (a.K & 7) == 0 && aligned16(a.x) &&
         (a.rms_w == nullptr || aligned16(a.rms_w)) &&
         (a.K_pad >> 3) <= kXKeep * kStagedThreads;
}

// Fast staging, first half: request x (and the norm weights with it: one memory round
// trip, not two).  Every request is unconditional per lane (an index past the end reads
// the last vector and is dropped at the use), so later code can wait for these loads by
// count while younger loads are still in flight.
__device__ __forceinline__ void x_request(const StreamArgs &a, uint4 (&v)[kXKeep],
                                          uint4 (&g)[kXKeep], uint4 &sq) {
  const int nk = a.K >> 3;
  const int deal = x_deal(a.K_pad >> 3);
  const int wave_first = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) & ~(kWave - 1));
  // (the parts of the sum of squares, or, without them, a vector of x that is dropped: a load
  // under a condition of its own would make the wait for x a wait for everything)
  sq = make_uint4(0, 0, 0, 0);
  if (wave_first < deal) {
    sq = a.sq_in != nullptr ? reinterpret_cast<const uint4 *>(a.sq_in)[threadIdx.x & (kWave - 1)]
                            : reinterpret_cast<const uint4 *>(a.x)[0];
  }
#pragma unroll
  for (int j = 0; j < kXKeep; ++j) {
    v[j] = make_uint4(0, 0, 0, 0);
    g[j] = make_uint4(0, 0, 0, 0);
    if (j * deal < nk && wave_first < deal) {
      const int i = min(static_cast<int>(threadIdx.x) + j * deal, nk - 1);
      v[j] = reinterpret_cast<const uint4 *>(a.x)[i];
      if (a.rms_w != nullptr) {
        g[j] = reinterpret_cast<const uint4 *>(a.rms_w)[i];
      }
    }
  }
}

// The inverse powers of two of the binary16 form, one float per pair of pieces (= per lane and
// half step, laid out [t][lane] like the lanes read them), behind the x pieces in LDS.
__device__ __forceinline__ float *x_factors(uint4 *xs, int K_pad) {
  return reinterpret_cast<float *>(xs + x_pieces(K_pad));
}

// One piece on its way to LDS: stored as it is, or (F16) as binary16 times the pair's power,
// whose inverse the pair's even thread leaves in the factor array.  Called by all lanes of a
// wavefront together (pair_power reads the neighbour lane); `live` says whether this thread
// has a piece to store.
template <bool F16>
__device__ __forceinline__ void store_piece(uint4 *xs, float *xf, int i, bool live, uint4 piece) {
  if constexpr (F16) {
    const int power = pair_power(live ? piece : make_uint4(0, 0, 0, 0));
    if (live) {
      xs[x_slot(i)] = piece_to_f16(piece, power);
      if ((i & 1) == 0) {
        xf[i >> 1] = __builtin_ldexpf(1.f, -power);
      }
    }
  } else {
    if (live) {
      xs[x_slot(i)] = piece;
    }
  }
}

// Fast staging, second half: normalise if asked, store the pieces, barrier.  With rms_w
// the value stored is bf16( (w*x) * rsqrt(mean(x^2)+eps) ), i.e. what a separate RMSNorm
// launch would have handed over (gpu/nf4/nf4_gemv.cu:264-289).  F16: those bf16 values are
// stored as binary16, pair by pair times a power of two (store_piece).
template <bool F16>
__device__ __forceinline__ void x_store(const StreamArgs &a, uint4 *xs, StagedLds &lds,
                                        const uint4 (&v)[kXKeep], const uint4 (&g)[kXKeep],
                                        const uint4 sq) {
  const int nk = a.K >> 3;
  const int nvec = a.K_pad >> 3;
  float *xf = x_factors(xs, a.K_pad);
  zero_unused_slots(xs, a.K_pad);
  if constexpr (F16) {
    // (the pairs of the last half step that no piece maps to: their lanes are switched off where
    // the scale is applied, but what they multiply must be finite)
    const int pairs = x_half_steps(a.K_pad) << 6;
    for (int h = (nvec + 1) / 2 + threadIdx.x; h < pairs; h += kStagedThreads) {
      xf[h] = 1.f;
    }
  }
  float inv = 1.f;
  // first vector index of this wavefront: a wavefront (or a round j of all of them) past the
  // end of x skips the arithmetic as a whole (a scalar branch) and only joins the barriers;
  // at K = 5120 eight wavefronts hold a vector, two of them a second one
  const int wave_first = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) & ~(kWave - 1));
  const int deal = x_deal(nvec);
  if (a.rms_w != nullptr && a.sq_in != nullptr) {
    // the writer of x left the sum in kSumsqParts parts: lane l holds parts 4l .. 4l+3 (only
    // the wavefronts that hold x need the factor; no barrier)
    if (wave_first < deal) {
      const float ss = wave_sum(((__uint_as_float(sq.x) + __uint_as_float(sq.y)) + __uint_as_float(sq.z)) +
                                __uint_as_float(sq.w));
      inv = rsqrtf(ss / static_cast<float>(a.K) + a.rms_eps);
    }
  } else if (a.rms_w != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kXKeep; ++j) {
      if (wave_first + j * deal >= nk || wave_first >= deal) {
        continue;
      }
      const int i = threadIdx.x + j * deal;
      const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
      float s4 = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        s4 = fmaf(bf16_lo(u[q]), bf16_lo(u[q]), s4);
        s4 = fmaf(bf16_hi(u[q]), bf16_hi(u[q]), s4);
      }
      ss += i < nk ? s4 : 0.f;
    }
    ss = block_sum(ss, lds.part);
    inv = rsqrtf(ss / static_cast<float>(a.K) + a.rms_eps);
  }
#pragma unroll
  for (int j = 0; j < kXKeep; ++j) {
    if (wave_first + j * deal >= nvec || wave_first >= deal) {
      continue;
    }
    const int i = threadIdx.x + j * deal;
    uint4 o = i < nk ? v[j] : make_uint4(0, 0, 0, 0);
    if (a.rms_w != nullptr) {
      const uint32_t u[4] = {o.x, o.y, o.z, o.w};
      const uint32_t gw[4] = {g[j].x, g[j].y, g[j].z, g[j].w};
      uint32_t r[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        r[q] = f32x2_to_bf16x2((bf16_lo(gw[q]) * bf16_lo(u[q])) * inv, (bf16_hi(gw[q]) * bf16_hi(u[q])) * inv);
      }
      o = make_uint4(r[0], r[1], r[2], r[3]);
    }
    store_piece<F16>(xs, xf, i, i < nvec, o);
  }
  __syncthreads();
}

// F16 staging of what the loops below left as bf16: every thread takes whole pairs of pieces.
__device__ __forceinline__ void staged_to_f16(const StreamArgs &a, uint4 *xs) {
  float *xf = x_factors(xs, a.K_pad);
  const int pairs = x_half_steps(a.K_pad) << 6;  // every slot pair of the staged half steps
  for (int h = threadIdx.x; h < pairs; h += kStagedThreads) {
    const int s0 = ((h >> 6) << 7) + (h & 63);  // slots of pieces 2 h and 2 h + 1
    const uint4 p0 = xs[s0], p1 = xs[s0 + 64];
    const uint32_t mask = 0x7FFF7FFFu;
    uint32_t m = pk_max_u16(pk_max_u16(pk_max_u16(p0.x & mask, p0.y & mask), pk_max_u16(p0.z & mask, p0.w & mask)),
                            pk_max_u16(pk_max_u16(p1.x & mask, p1.y & mask), pk_max_u16(p1.z & mask, p1.w & mask)));
    m = max(m & 0xFFFFu, m >> 16);
    const int power = (m == 0u || m >= 0x7F80u) ? 0 : 14 - (static_cast<int>(m >> 7) - 127);
    xs[s0] = piece_to_f16(p0, power);
    xs[s0 + 64] = piece_to_f16(p1, power);
    xf[h] = __builtin_ldexpf(1.f, -power);
  }
  __syncthreads();
}

// Staging for the other cases: the attention merge, a ragged K, unaligned pointers.
template <bool F16>
__device__ __forceinline__ void stage_x(const StreamArgs &a, uint4 *xs, StagedLds &lds) {
  float *part = lds.part;
  zero_unused_slots(xs, a.K_pad);
  if (a.attn_state != nullptr) {
    const int nvec = a.K_pad >> 3;
    if (nvec <= kStagedThreads && (nvec & 127) == 0) {
      // one piece a thread at most (K <= 8192, whole half steps): it stays in registers from
      // the merge to the store
      float *xf = x_factors(xs, a.K_pad);
      const int i = threadIdx.x;
      const int wave_first = __builtin_amdgcn_readfirstlane(i & ~(kWave - 1));
      if (wave_first < nvec) {
        const uint4 piece = a.attn_parts <= 4 ? merged_attn_piece<4>(a, i) : merged_attn_piece<8>(a, i);
        store_piece<F16>(xs, xf, i, true, piece);
      }
      __syncthreads();
      return;
    }
    for (int i = threadIdx.x; i < nvec; i += kStagedThreads) {
      xs[x_slot(i)] = a.attn_parts <= 4 ? merged_attn_piece<4>(a, i) : merged_attn_piece<8>(a, i);
    }
    __syncthreads();
    if constexpr (F16) {
      staged_to_f16(a, xs);
    }
    return;
  }
  {
    float inv = 1.f;
    if (a.rms_w != nullptr) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < a.K; i += kStagedThreads) {
        const float v = bf16_to_f32(a.x[i]);
        ss = fmaf(v, v, ss);
      }
      ss = block_sum(ss, part);
      inv = rsqrtf(ss / static_cast<float>(a.K) + a.rms_eps);
    }
    uint16_t *xh = reinterpret_cast<uint16_t *>(xs);
    for (int i = threadIdx.x; i < a.K_pad; i += kStagedThreads) {
      uint16_t v = 0;
      if (i < a.K) {
        v = a.x[i];
        if (a.rms_w != nullptr) {
          v = f32_to_bf16((bf16_to_f32(a.rms_w[i]) * bf16_to_f32(v)) * inv);
        }
      }
      xh[(x_slot(i >> 3) << 3) + (i & 7)] = v;
    }
  }
  __syncthreads();
  if constexpr (F16) {
    staged_to_f16(a, xs);
  }
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

constexpr int kStagedSmallBytes = 512;  // GemvLds of a staged kernel, after the table
static_assert(sizeof(StagedLds) <= kStagedSmallBytes, "the small statics must fit their slot");

typedef __attribute__((ext_vector_type(2))) __bf16 Bf16x2;

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(Bf16x2, a),
                                         __builtin_bit_cast(Bf16x2, b), acc, false);
}

typedef __attribute__((ext_vector_type(2))) _Float16 F16x2v;

__device__ __forceinline__ float dot2_f16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(F16x2v, a), __builtin_bit_cast(F16x2v, b), acc, false);
}

// Products of one level pair with one pair of x for the single-lookup forms: bf16 levels times
// bf16 x (LEVELS 1), binary16 levels times x staged as binary16 (LEVELS 3).
template <int LEVELS>
__device__ __forceinline__ float dot2_levels(uint32_t a, uint32_t b, float acc) {
  if constexpr (LEVELS == 3) {
    return dot2_f16(a, b, acc);
  } else {
    return dot2_bf16(a, b, acc);
  }
}

// ---- binary16 pair table --------------------------------------------------------------
// The pair table of nf4_common.h with the levels rounded to binary16 instead of bf16: 11
// significant bits, 2^-12 relative weight error against 2^-9, same table size, same single
// 4-byte lookup per two weights.  Filled by a workgroup of exactly 16 wavefronts.
constexpr uint32_t f16_bits_rne(uint32_t b) {  // finite, zero or of a magnitude binary16 holds as a normal number
  if ((b & 0x7FFFFFFFu) == 0u) {
    return (b >> 16) & 0x8000u;
  }
  uint32_t half = ((b >> 16) & 0x8000u) | ((((b >> 23) & 0xFFu) - 112u) << 10) | ((b & 0x7FFFFFu) >> 13);
  const uint32_t rem = b & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u) != 0u)) {
    ++half;
  }
  return half;
}

__device__ __forceinline__ void fill_pair_table_f16(uint32_t *table, int wave, int lane) {
  const uint32_t lo = __builtin_bit_cast(uint16_t, static_cast<_Float16>(bits_to_f32(kLutBits[wave])));
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const uint32_t hi = f16_bits_rne(kLevelBits[j]) << 16;
    table[((wave + 16 * j) << 6) + lane] = lo | hi;
  }
}

// ---- two-term pair table ----------------------------------------------------------------
// A level is kept as the sum of two bf16 values: head = bf16(level) and tail =
// bf16(level - head), 16 to 17 significant bits together, so the products with bf16
// activations are exact and the weight error falls from 2^-9 to below 2^-17 relative: under
// the rounding of an fp32 accumulation over a row.  An entry is 8 bytes {head pair, tail
// pair}; 32 copies (lane & 31) make the 64-bit reads conflict-free (the LDS serves a
// ds_read_b64 half a wavefront at a time), so the table is still 64 KB and a lookup is
// still one v_perm_b32 (byte 1 = the packed byte, byte 0 = 8 * (lane & 31)) and one LDS
// read; the second term costs one more v_dot2c_f32_bf16 per pair.
constexpr uint32_t level_tail_bf16(uint32_t level_bits) {
  const float level = __builtin_bit_cast(float, level_bits);
  const float head = __builtin_bit_cast(float, bf16_bits_rne(level_bits) << 16);
  return bf16_bits_rne(__builtin_bit_cast(uint32_t, level - head));
}

// Filled by a workgroup of exactly 16 wavefronts.  Wavefront v owns the bytes whose low
// code is v; lanes 0..31 write the copies of high code 2jj, lanes 32..63 those of 2jj+1.
__device__ __forceinline__ void fill_pair2_table(uint2 *table, int wave, int lane) {
  const uint32_t lo_h = bf16_bits_rne(kLutBits[wave]);
  const uint32_t lo_t = level_tail_bf16(kLutBits[wave]);
  const int copy = lane & 31;
  const bool odd = lane >= 32;
#pragma unroll
  for (int jj = 0; jj < 8; ++jj) {
    const int j = 2 * jj + (odd ? 1 : 0);
    const uint32_t hi_h = odd ? bf16_bits_rne(kLevelBits[2 * jj + 1]) : bf16_bits_rne(kLevelBits[2 * jj]);
    const uint32_t hi_t = odd ? level_tail_bf16(kLevelBits[2 * jj + 1]) : level_tail_bf16(kLevelBits[2 * jj]);
    table[((wave + 16 * j) << 5) + copy] = make_uint2(lo_h | (hi_h << 16), lo_t | (hi_t << 16));
  }
}

__device__ __forceinline__ uint2 lds0_u64(uint32_t addr) {
  const U32x2 v = *reinterpret_cast<const __attribute__((address_space(3))) U32x2 *>(addr);
  return make_uint2(v.x, v.y);
}

template <int J>
__device__ __forceinline__ uint2 pair2_at(uint32_t w, uint32_t lane8) {
  constexpr uint32_t sel = 0x0C0C0400u + (static_cast<uint32_t>(J) << 8);
  return lds0_u64(__builtin_amdgcn_perm(w, lane8, sel));
}

// One wavefront, R weight rows sharing x, which is read from global memory (K_pad/8
// 16-byte pieces at x4).
template <int R>
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
        const uint4 v = stream_load16(reinterpret_cast<const uint4 *>(prow[r]) + c);
        w[r][0] = v.x;
        w[r][1] = v.y;
        w[r][2] = v.z;
        w[r][3] = v.w;
        sc[r] = stream_load2(srow[r] + (c >> 1));
      }
      const uint4 *xp = x4 + (c << 2);
      const uint4 x0 = xp[0], x1 = xp[1], x2 = xp[2], x3 = xp[3];
      float xf[32];
      widen8(x0, xf);
      widen8(x1, xf + 8);
      widen8(x2, xf + 16);
      widen8(x3, xf + 24);
      rows_step<R, 4>(w, xf, sc, lut, acc);
    } else {
      const int h = ((t - nfull) << 6) + lane;
      if (h < tail_half) {
        const int hc = base_half + h;  // half-chunk index in the row: 16 weights
        uint32_t w[R][2];
        uint16_t sc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint2 v = stream_load8(reinterpret_cast<const uint2 *>(prow[r]) + hc);
          w[r][0] = v.x;
          w[r][1] = v.y;
          sc[r] = stream_load2(srow[r] + (hc >> 2));
        }
        const uint4 *xp = x4 + (hc << 1);
        const uint4 x0 = xp[0], x1 = xp[1];
        float xf[16];
        widen8(x0, xf);
        widen8(x1, xf + 8);
        rows_step<R, 2>(w, xf, sc, lut, acc);
      }
    }
  }
}

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }

// Segment, first row and row count of a row group numbered through the segments.
template <bool SWIGLU>
__device__ __forceinline__ void group_rows(const StreamArgs &a, int grp, int U, int &seg,
                                           int &row0, int &M) {
  int g = grp;
  seg = 0;
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
  M = a.M[seg];
  row0 = g * U;
}

template <int R, bool SWIGLU>
__device__ __forceinline__ void group_pointers(const StreamArgs &a, int grp,
                                               const uint8_t *(&prow)[R],
                                               const uint16_t *(&srow)[R]) {
  constexpr int U = SWIGLU ? R / 2 : R;
  int seg, row0, M;
  group_rows<SWIGLU>(a, grp, U, seg, row0, M);
  const size_t pstride = static_cast<size_t>(a.K_pad >> 1);
  const size_t sstride = static_cast<size_t>(a.K_pad >> 6);
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
}

// Plain kernel: four wavefronts per workgroup, x read from global memory.
// SWIGLU == false: R rows of one segment per wavefront, epilogue y = acc (+ add).
// SWIGLU == true : R/2 gate rows and the matching R/2 up rows per wavefront,
//                  epilogue y = silu(gate) * up from the unrounded fp32 sums.
template <int R, bool SWIGLU>
__global__ __launch_bounds__(256) void gemv_stream(const StreamArgs a) {
  __shared__ GemvLds lds;
  constexpr int U = SWIGLU ? R / 2 : R;  // output rows per wavefront
  const int lane = threadIdx.x & (kWave - 1);
  // The wavefront index is the same in every lane: saying so keeps the row-group and
  // segment arithmetic, and the kernel-argument reads indexed by it, on the scalar unit.
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  constexpr int waves = kThreads >> 6;  // (every launch of this kernel has kThreads threads)

  if (threadIdx.x < 16) {
    lds.lut[threadIdx.x] = bits_to_f32(kLutBits[threadIdx.x]);
  }
  // Row groups (U rows each) are numbered through the segments; a wavefront takes exactly
  // one group, or, with ksplit, the wavefronts of a workgroup share one along K.
  const int total = a.groups[0] + a.groups[1] + a.groups[2];
  const bool ksplit = !SWIGLU && a.ksplit > 1;
  const int grp = ksplit ? static_cast<int>(blockIdx.x)
                         : static_cast<int>(blockIdx.x) * waves + wave;
  __syncthreads();
  if (grp >= total) {
    return;
  }
  int seg, row0, M;
  group_rows<SWIGLU>(a, grp, U, seg, row0, M);
  const uint8_t *prow[R];
  const uint16_t *srow[R];
  group_pointers<R, SWIGLU>(a, grp, prow, srow);

  float acc[R] = {};
  rows_dot<R>(prow, srow, reinterpret_cast<const uint4 *>(a.x), a.K_pad, lds.lut, lane, acc,
              ksplit ? wave : 0, ksplit ? waves : 1);

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
      const float sv = sums[u];
      const int r = row0 + u;
      if (writer && lane == u && r < M) {
        float v = sv;
        if (add != nullptr) {
          v += bf16_to_f32(add[r]);
        }
        y[r] = f32_to_bf16(v);
      }
    }
  }
}

// The level table of a kernel that stages x in LDS, by the form of its levels.
template <int TERMS>
__device__ __forceinline__ void fill_level_table(uint4 *dyn_lds, int wave, int lane) {
  if constexpr (TERMS == 1) {
    fill_pair_table(reinterpret_cast<uint32_t *>(dyn_lds), wave, lane);
  } else if constexpr (TERMS == 3) {
    fill_pair_table_f16(reinterpret_cast<uint32_t *>(dyn_lds), wave, lane);
  } else {
    fill_pair2_table(reinterpret_cast<uint2 *>(dyn_lds), wave, lane);
  }
}

// ---- staged kernel: x in LDS, pair table, weight requests one item ahead -----------
// Request half step t of R rows: 8 packed bytes per lane.  Lanes past the end of the row
// read the row's last half chunk instead (in bounds, one instruction form for every
// step) and are switched off where the scale is applied.
template <int R>
__device__ __forceinline__ void load_step(const uint8_t *const (&prow)[R],
                                          const uint16_t *const (&srow)[R], int n_half, int t,
                                          int lane, uint2 (&w)[R], uint16_t (&sc)[R]) {
  const int h = min((t << 6) + lane, n_half - 1);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    w[r] = stream_load8(reinterpret_cast<const uint2 *>(prow[r]) + h);
    sc[r] = stream_load2(srow[r] + (h >> 2));
  }
}

// TERMS == 1: levels as one bf16 (pair table of dwords, 64 copies).  TERMS == 2: levels as
// head + tail (two-term table, 32 copies of 8-byte entries).  TERMS == 3: levels as one
// binary16 against x staged as binary16 (same table shape as TERMS == 1).
template <int R, int TERMS>
__device__ __forceinline__ void dot_step(const uint2 (&w)[R], const uint16_t (&sc)[R],
                                         const uint4 *xs, const float *xf, int n_half, int t, int lane,
                                         float (&acc)[R]) {
  const bool on = (t << 6) + lane < n_half;
  // binary16 x: the inverse of the power of two this lane's 16 activations were staged with
  const float factor = TERMS == 3 ? xf[(t << 6) + lane] : 1.f;
  const uint4 *xp = xs + (t << 7) + lane;
  const uint4 x0 = xp[0], x1 = xp[64];
  if constexpr (TERMS != 2) {
    const uint32_t lane4 = static_cast<uint32_t>(lane) << 2;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float pa = 0.f, pb = 0.f;
      pa = dot2_levels<TERMS>(pair_at<0>(w[r].x, lane4), x0.x, pa);
      pb = dot2_levels<TERMS>(pair_at<1>(w[r].x, lane4), x0.y, pb);
      pa = dot2_levels<TERMS>(pair_at<2>(w[r].x, lane4), x0.z, pa);
      pb = dot2_levels<TERMS>(pair_at<3>(w[r].x, lane4), x0.w, pb);
      pa = dot2_levels<TERMS>(pair_at<0>(w[r].y, lane4), x1.x, pa);
      pb = dot2_levels<TERMS>(pair_at<1>(w[r].y, lane4), x1.y, pb);
      pa = dot2_levels<TERMS>(pair_at<2>(w[r].y, lane4), x1.z, pa);
      pb = dot2_levels<TERMS>(pair_at<3>(w[r].y, lane4), x1.w, pb);
      const float scale = on ? f16_to_f32(sc[r]) * factor : 0.f;
      acc[r] = fmaf(scale, pa + pb, acc[r]);
    }
  } else {
    const uint32_t lane8 = static_cast<uint32_t>(lane & 31) << 3;
    const uint32_t xw[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint2 e[8] = {pair2_at<0>(w[r].x, lane8), pair2_at<1>(w[r].x, lane8),
                          pair2_at<2>(w[r].x, lane8), pair2_at<3>(w[r].x, lane8),
                          pair2_at<0>(w[r].y, lane8), pair2_at<1>(w[r].y, lane8),
                          pair2_at<2>(w[r].y, lane8), pair2_at<3>(w[r].y, lane8)};
      // heads and tails in separate sums: the tails are 2^-9 of the heads and would lose
      // their low bits if they were added into the large sum one by one
      float ha = 0.f, hb = 0.f, ta = 0.f, tb = 0.f;
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        ha = dot2_bf16(e[j].x, xw[j], ha);
        ta = dot2_bf16(e[j].y, xw[j], ta);
        hb = dot2_bf16(e[j + 1].x, xw[j + 1], hb);
        tb = dot2_bf16(e[j + 1].y, xw[j + 1], tb);
      }
      const float scale = on ? f16_to_f32(sc[r]) : 0.f;
      acc[r] = fmaf(scale, (ha + hb) + (ta + tb), acc[r]);
    }
  }
}

// bf16 at a wavefront-uniform address, read on the scalar unit as the aligned dword that
// holds it: the read then does not join the in-order queue of vector loads, so taking it
// does not wait for weights requested ahead.
__device__ __forceinline__ float uniform_bf16(const uint16_t *p) {
  typedef const __attribute__((address_space(4))) uint32_t *ScalarWord;
  const uintptr_t u = reinterpret_cast<uintptr_t>(p);
  const uint32_t word = *reinterpret_cast<ScalarWord>(u & ~static_cast<uintptr_t>(3));
  return (u & 2) != 0 ? bf16_hi(word) : bf16_lo(word);
}

// One workgroup of 16 wavefronts per compute unit; a wavefront walks the row groups
// wave*grid + block, + 16*grid, ..  The half steps of those groups, in order, are the
// wavefront's work list; an item is S consecutive ones (it may span two groups).  The S
// requests of an item are issued back to back into one of two register buffers; while item i is
// computed from one buffer, item i+1 is already in flight into the other, across group
// borders too, so a wavefront always has S*R*8 bytes per lane on the way.  Between a
// request and its use the code is straight-line (the loop is written out for both buffer
// parities and the last item has its own copy without a request), so the wait counts the
// compiler derives are exact: step j waits for its own data while steps j+1.. and the
// whole next item are still arriving.  The first item is requested before x is staged:
// the weight stream starts with the kernel.
//   SWIGLU == false: R rows of one segment per group, epilogue y = acc (+ add).
//   SWIGLU == true : R/2 gate rows and the matching R/2 up rows, y = silu(gate) * up
//                    from the unrounded fp32 sums.
template <int R, int S, bool SWIGLU, int TERMS>
__global__ __launch_bounds__(1024) void gemv_staged(const StreamArgs a) {
  extern __shared__ uint4 dyn_lds[];  // [pair table][GemvLds][x pieces], table at address 0
  char *base = reinterpret_cast<char *>(dyn_lds);
  StagedLds &lds = *reinterpret_cast<StagedLds *>(base + kPairTableBytes);
  uint4 *xs = reinterpret_cast<uint4 *>(base + kPairTableBytes + kStagedSmallBytes);
  const float *xf = x_factors(xs, a.K_pad);
  constexpr int U = SWIGLU ? R / 2 : R;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  constexpr int waves = kStagedThreads >> 6;
  const int total = a.groups[0] + a.groups[1] + a.groups[2];
  // (the grid size and how the groups split into passes come from the host: read from the
  // hidden kernel arguments and divided here they were a trip to the scalar cache and an integer
  // division ahead of the first requests)
  const int first = wave * a.ring_grid + static_cast<int>(blockIdx.x);
  const int stride = a.ring_grid * waves;
  const int n_half = a.K_pad >> 4;
  const int nsteps = x_half_steps(a.K_pad);
  const int my_groups = a.ring_passes + (first < a.ring_left ? 1 : 0);
  const int n_steps_all = my_groups * nsteps;      // half steps of this wavefront, in order
  const int n_items = (n_steps_all + S - 1) / S;   // S of them per item, across group borders

  // request cursor: half step pi of the list = step pt of group pg
  int pi = 0, pg = first, pt = 0;
  const uint8_t *prow[R];
  const uint16_t *srow[R];
  uint2 wa[S][R], wb[S][R];
  uint16_t sa[S][R], sb[S][R];

  // Past the end of the list the cursor stays on the last half step: the repeat is
  // served by the cache and keeps the number of loads per item fixed.
#define CHR_REQUEST(W, SC)                                              \
  _Pragma("unroll") for (int j = 0; j < S; ++j) {                       \
    load_step<R>(prow, srow, n_half, pt, lane, W[j], SC[j]);            \
    if (pi + 1 < n_steps_all) {                                         \
      ++pi;                                                             \
      if (++pt == nsteps) {                                             \
        pt = 0;                                                         \
        pg += stride;                                                   \
        group_pointers<R, SWIGLU>(a, pg, prow, srow);                   \
      }                                                                 \
    }                                                                   \
  }

  auto fill_table = [&]() { fill_level_table<TERMS>(dyn_lds, wave, lane); };

  // Order of the first requests: x, then the first item of weights, and only then the
  // wait for x.  Vector loads return in order, so x must be the older request or its wait
  // would be a wait for the weights too.  Each case below is its own straight-line path
  // (the two copies of the stores and barriers are the price): a path that merged
  // "weights requested" with "nothing requested" would make the wait a wait for all.
  if (stage_fast_ok(a)) {
    uint4 xv[kXKeep], xg[kXKeep], xq;
    x_request(a, xv, xg, xq);
    if (n_items > 0) {
      group_pointers<R, SWIGLU>(a, first, prow, srow);
      CHR_REQUEST(wa, sa)
      fill_table();
      x_store<TERMS == 3>(a, xs, lds, xv, xg, xq);
    } else {
      fill_table();
      x_store<TERMS == 3>(a, xs, lds, xv, xg, xq);
    }
  } else {
    // The other staging forms read what they need in loops of their own; the first item
    // is requested ahead of them all the same: its trip to memory (the long one) then
    // overlaps the staging, at the price of the staging's first loads returning behind it.
    if (n_items > 0) {
      group_pointers<R, SWIGLU>(a, first, prow, srow);
      CHR_REQUEST(wa, sa)
    }
    fill_table();
    stage_x<TERMS == 3>(a, xs, lds);
  }

  // compute cursor: half step ci of the list = step ct of group cg
  int ci = 0, cg = first, ct = 0;
  float acc[R] = {};
  float sq_acc = 0.f;  // sq_out: sum of squares of what this wavefront has stored

  auto finish_group = [&](int grp) {
    int seg, row0, M;
    group_rows<SWIGLU>(a, grp, U, seg, row0, M);
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
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float v = wave_sum(acc[u]);
        const int r = row0 + u;
        if (add != nullptr) {
          v += uniform_bf16(add + min(r, M - 1));
        }
        const uint16_t stored = f32_to_bf16(v);
        if (lane == u && r < M) {
          y[r] = stored;
        }
        if (a.sq_out != nullptr && r < M) {
          const float rf = bf16_to_f32(stored);
          sq_acc = fmaf(rf, rf, sq_acc);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = 0.f;
    }
  };

#define CHR_COMPUTE(W, SC)                                              \
  _Pragma("unroll") for (int j = 0; j < S; ++j) {                       \
    if (ci < n_steps_all) {                                             \
      dot_step<R, TERMS>(W[j], SC[j], xs, xf, n_half, ct, lane, acc);          \
      ++ci;                                                             \
      if (++ct == nsteps) {                                             \
        finish_group(cg);                                               \
        ct = 0;                                                         \
        cg += stride;                                                   \
      }                                                                 \
    }                                                                   \
  }

  if (n_items > 0) {
    int i = 0;
    while (true) {
      // item i is in (wa, sa)
      if (i + 1 >= n_items) {
        CHR_COMPUTE(wa, sa)
        break;
      }
      CHR_REQUEST(wb, sb)
      CHR_COMPUTE(wa, sa)
      ++i;
      // item i is in (wb, sb)
      if (i + 1 >= n_items) {
        CHR_COMPUTE(wb, sb)
        break;
      }
      CHR_REQUEST(wa, sa)
      CHR_COMPUTE(wb, sb)
      ++i;
    }
  }
#undef CHR_COMPUTE
#undef CHR_REQUEST
  if constexpr (!SWIGLU) {
    if (a.sq_out != nullptr) {
      store_sumsq_part(a, lds, sq_acc, wave, lane);
    }
  }
}

// ---- ring kernel: weight requests and their waits written by hand ----------------------
// The staged kernel above leaves the software pipeline to the compiler, whose wait counts
// turn conservative wherever paths with different loads in flight meet (a loop head, the
// join after a branch): how deep a pipeline it keeps then depends on register allocation.
// Here the weight requests, the waits for them and the first instructions that read them
// are asm, and the registers they go through are fixed ones above the compiler's VGPR
// budget (nf4_gemv_ring_regs.h), which it therefore never touches.  Vector memory
// operations complete in order, so "at most N outstanding" means everything but the N
// youngest has arrived: every wait below is exact by construction.
//
// NS slots of one half step each form a ring: while the oldest is computed, NS-1-LAG younger
// ones are in flight; a slot is free once its bytes have been turned into lookup addresses
// and is requested again LAG steps later (LAG is chosen per ring length in the body).  Work is
// dealt as in the staged kernel's comment.
struct XRegs {
  U32x4 v[kXKeep];  // x, 16-byte vectors i = thread + j * x_deal()
  U32x4 g[kXKeep];  // the RMSNorm weights at the same places (fused norm only)
  U32x4 q;          // four of the sum-of-squares parts a writer left (sq_in only)
};

// A request whose destination keeps its value where the request is skipped: in/out operand,
// so both paths hold it in the same registers and nothing is copied while it is in flight.
__device__ __forceinline__ void request16(U32x4 &d, const void *p, uint32_t &tok) {
  asm("global_load_dwordx4 %0, %2, off" : "+v"(d), "+s"(tok) : "v"(p));
}

__device__ __forceinline__ void ring_x_request(const StreamArgs &a, XRegs &x, uint32_t &tok) {
  const int nk = a.K >> 3;
  const int deal = x_deal(a.K_pad >> 3);
  const int wave_first = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) & ~(kWave - 1));
  x.q = U32x4{0u, 0u, 0u, 0u};
  if (a.sq_in != nullptr && wave_first < deal) {
    request16(x.q, reinterpret_cast<const uint4 *>(a.sq_in) + (threadIdx.x & (kWave - 1)), tok);
  }
#pragma unroll
  for (int j = 0; j < kXKeep; ++j) {
    x.v[j] = U32x4{0u, 0u, 0u, 0u};
    x.g[j] = U32x4{0u, 0u, 0u, 0u};
    if (j * deal < nk && wave_first < deal) {
      const int i = min(static_cast<int>(threadIdx.x) + j * deal, nk - 1);
      request16(x.v[j], reinterpret_cast<const uint4 *>(a.x) + i, tok);
      if (a.rms_w != nullptr) {
        request16(x.g[j], reinterpret_cast<const uint4 *>(a.rms_w) + i, tok);
      }
    }
  }
}

// x has arrived once at most YOUNGER vector memory operations are outstanding.
template <int YOUNGER>
__device__ __forceinline__ void ring_x_wait(XRegs &x, uint32_t &tok) {
  static_assert(kXKeep == 4, "operand list below");
  asm("s_waitcnt vmcnt(%10) ; covers %0 %1 %2 %3 %4 %5 %6 %7 %8"
      : "+v"(x.v[0]), "+v"(x.v[1]), "+v"(x.v[2]), "+v"(x.v[3]), "+v"(x.g[0]), "+v"(x.g[1]),
        "+v"(x.g[2]), "+v"(x.g[3]), "+v"(x.q), "+s"(tok)
      : "n"(YOUNGER));
}

// The eight lookup addresses of one half step of one row (v_perm_b32: byte 1 = a packed
// byte, byte 0 = the lane's offset into its table copy) and the row's scale as fp32, read
// from the fixed registers X, Y (packed dwords) and S (fp16 scale, zero-extended).
//
// None of the ring's asm statements is volatile: a volatile asm orders every LDS and global
// access of the compiler's around it, which serialises a half step (x reads, lookups and
// products of neighbouring steps could no longer overlap: measured 15 against 10 us).
// Instead every statement reads and writes one scalar token, TOK, which chains them in
// program order among themselves and keeps them out of common-subexpression and
// loop-invariant motion, while the compiler's own memory operations move freely.
#define CHR_RING_ADDRESSES(X, Y, S, A, SC, LANE_OFF, TOK)                                 \
  asm("v_perm_b32 %0, " X ", %10, %11\n\t"                                                \
      "v_perm_b32 %1, " X ", %10, %12\n\t"                                                \
      "v_perm_b32 %2, " X ", %10, %13\n\t"                                                \
      "v_perm_b32 %3, " X ", %10, %14\n\t"                                                \
      "v_perm_b32 %4, " Y ", %10, %11\n\t"                                                \
      "v_perm_b32 %5, " Y ", %10, %12\n\t"                                                \
      "v_perm_b32 %6, " Y ", %10, %13\n\t"                                                \
      "v_perm_b32 %7, " Y ", %10, %14\n\t"                                                \
      "v_cvt_f32_f16 %8, " S                                                              \
      : "=&v"(A[0]), "=&v"(A[1]), "=&v"(A[2]), "=&v"(A[3]), "=&v"(A[4]), "=&v"(A[5]),     \
        "=&v"(A[6]), "=&v"(A[7]), "=&v"(SC), "+s"(TOK)                                    \
      : "v"(LANE_OFF), "s"(0x0C0C0400u), "s"(0x0C0C0500u), "s"(0x0C0C0600u),              \
        "s"(0x0C0C0700u))

// One row's half step from its eight lookup addresses: products of level pairs with the
// bf16 pairs of x (xw), the scale applied to the 16-weight partial.
template <int TERMS>
__device__ __forceinline__ float ring_row_dot(const uint32_t (&adr)[8], const uint32_t (&xw)[8]) {
  if constexpr (TERMS != 2) {
    float pa = 0.f, pb = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      pa = dot2_levels<TERMS>(lds0_u32(adr[j]), xw[j], pa);
      pb = dot2_levels<TERMS>(lds0_u32(adr[j + 1]), xw[j + 1], pb);
    }
    return pa + pb;
  } else {
    uint2 e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      e[j] = lds0_u64(adr[j]);
    }
    // heads and tails in separate sums: the tails are 2^-9 of the heads and would lose
    // their low bits if they were added into the large sum one by one
    float ha = 0.f, hb = 0.f, ta = 0.f, tb = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      ha = dot2_bf16(e[j].x, xw[j], ha);
      ta = dot2_bf16(e[j].y, xw[j], ta);
      hb = dot2_bf16(e[j + 1].x, xw[j + 1], hb);
      tb = dot2_bf16(e[j + 1].y, xw[j + 1], tb);
    }
    return (ha + hb) + (ta + tb);
  }
}

// The loop is written for instruction count as much as for memory: at four wavefronts per
// SIMD a half step of ~70 instructions (what the compiler-pipelined kernel executes, half of
// it address arithmetic and cursor bookkeeping) makes the launch issue-bound, not HBM-bound.
// Here a row is walked in pieces of NS half steps with NS a compile-time constant, one ring
// slot per half step of a piece: a request is two instructions whose row and piece live in a
// scalar base pointer and whose half step is an immediate offset, the x pieces are read at
// immediate offsets from one address per piece, and the cursors only move where a piece ends.
//
// Work is dealt by whole groups: wavefront w of workgroup b walks groups w*grid + b,
// + 16*grid, ..; after the last full pass the first wavefronts take one more.  (Dealing the
// left-over groups out by half steps, sums meeting in LDS, made all wavefronts finish
// together and the launch slower: 10.8 against 10.3 us at 13824x5120 -- while the last
// groups run, the fewer wavefronts still at work are served faster.)
//
// PAD: a row whose half steps are not a multiple of NS ends in a piece with PAD slots too
// many.  Those slots are requested like the others (a fixed number of requests per piece is
// what makes the waits exact), from the piece's first half step, which is there and cached,
// and never computed.
//
// SEQ (single rows): a group is a gate row and the up row of the same index, walked one after
// the other through the same ring (same x, same registers as a plain row); the gate's sum
// waits in a register for the up row's, and the pair leaves silu(gate) * up.
template <int NS, int TERMS, bool XREG, int PAD = 0, bool SEQ = false>
__device__ __forceinline__ void gemv_ring_body(const StreamArgs &a) {
  static_assert(NS >= 2 && NS <= 8, "slots of the ring that have registers");
  static_assert(!XREG || NS <= 5, "x of a whole row in 8 * NS registers");
  static_assert(PAD >= 0 && PAD < NS && !(XREG && PAD > 0), "slots left empty in a row's last piece");
  constexpr int kLastReal = NS - 1 - PAD;  // last slot of a row's last piece that holds a half step
  constexpr int R = 1;                 // rows in the ring at a time
  constexpr int D = NS;                // slots of the ring
  constexpr int kStepLoads = 2 * R;    // vector memory operations of one half step
  // A slot is requested again LAG steps after the step that consumed it, so NS - LAG half steps
  // of a wavefront are in flight or being computed, not NS: this memory system serves a launch
  // fastest with about 2 KB per wavefront on the way (ring_piece_steps), a half step is 544
  // bytes.  Measured, us per launch at lag 0 / 1 / 2 / 3 (a dash: not measured): five slots
  // 13824x5120 9.11 / 8.76 / 9.05 / -, 152064x5120 69.3 / 68.4 / 67.0 / -; six slots 8192x6144
  // - / 7.98 / 7.21 / 7.28, 16384x6144 - / 12.8 / 11.6 .. 12.3 / 11.7, 20B decode 324 / - / 333 /
  // 336 tok/s; seven slots 5120x13824 - / 10.06 / 9.52 / 9.59, 8192x7168 - / 9.65 / 8.63 / 8.01,
  // 5120x27648 - / 16.1 / 16.2 / 16.9; four slots 8192x4096 6.00 / 5.90, 6144x16384 11.9 / 12.3.
  // 14B decode 392 -> 399 tok/s, 20B 324 -> 336.
  constexpr int LAG = NS == 4 ? 0 : NS == 5 ? 1 : NS == 6 ? 3 : NS == 7 ? 2 : 3;
  static_assert(LAG >= 0 && LAG < NS - 2, "at least two half steps in flight");
  // LDS byte address of the x pieces (the pair table starts at LDS address 0)
  constexpr uint32_t kXsAddr = kPairTableBytes + kStagedSmallBytes;
  extern __shared__ uint4 dyn_lds[];  // [pair table][GemvLds][x pieces]
  char *base = reinterpret_cast<char *>(dyn_lds);
  StagedLds &lds = *reinterpret_cast<StagedLds *>(base + kPairTableBytes);
  uint4 *xs = reinterpret_cast<uint4 *>(base + kXsAddr);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  uint32_t tok = 0;  // orders the asm statements among themselves, see CHR_RING_ADDRESSES

  // Group g is row g of the segments laid end to end (one segment for a plain GEMV, three
  // for q/k/v), or gate row g and up row g.  How the groups split into full passes and
  // left-over ones is the same for every wavefront and comes from the host.
  constexpr int waves = kStagedThreads >> 6;
  const int grid = a.ring_grid;
  const int block = static_cast<int>(blockIdx.x);
  const int first = wave * grid + block;
  const int stride = grid * waves;
  const int n_half = a.K_pad >> 4;
  const int nsteps = x_half_steps(a.K_pad);   // pieces * NS - PAD (the host's choice of both)
  const int pieces = (nsteps + PAD) / NS;     // pieces of a row
  const int last_t = nsteps - 1;
  const int rem = n_half - last_t * kWave;  // lanes of a row's last half step that hold a chunk
  const bool ragged = rem < kWave;
  const uint64_t row_bytes = static_cast<uint64_t>(a.K_pad >> 1);
  const uint64_t row_scale_bytes = static_cast<uint64_t>(a.K_pad >> 6) << 1;
  const int seg_end0 = a.groups[0];
  const int seg_end1 = a.groups[0] + a.groups[1];
  const bool one_segment = SEQ || a.groups[1] + a.groups[2] == 0;

  // per-lane loop constants: byte offsets into a half step of packed bytes / of scales (and
  // their clamped forms for a ragged last step), the x pieces' LDS address, the lane's copy
  // of the level table
  const uint32_t v_w = static_cast<uint32_t>(lane) << 3;
  const uint32_t v_s = static_cast<uint32_t>(lane >> 2) << 1;
  const uint32_t v_wl = static_cast<uint32_t>(min(lane, rem - 1)) << 3;
  const uint32_t v_sl = static_cast<uint32_t>(min(lane, rem - 1) >> 2) << 1;
  const uint32_t x_lane = kXsAddr + (static_cast<uint32_t>(lane) << 4);
  // binary16 x: the lane's inverse powers, one float per half step, behind the x pieces
  const uint32_t f_lane = kXsAddr + (static_cast<uint32_t>(x_pieces(a.K_pad)) << 4) +
                          (static_cast<uint32_t>(lane) << 2);
  const uint32_t lane_off = TERMS != 2 ? static_cast<uint32_t>(lane) << 2
                                       : static_cast<uint32_t>(lane & 31) << 3;
  const uint64_t last_lanes = ragged ? ((uint64_t{1} << rem) - 1) : ~uint64_t{0};

  // Set-up is written for the number of scalar instructions ahead of the first requests:
  // the 16 wavefronts of a workgroup start together and share four scalar units, so every
  // instruction here costs four cycles of every wavefront's start.
  const int my_groups = a.ring_passes + (first < a.ring_left ? 1 : 0);

  // ---- request cursor: piece q_part of group q_group at wq / sq --------------------------
  uint64_t wq[R], sq[R];
  constexpr int kRowsPerGroup = SEQ ? 2 : 1;
  int q_left = my_groups * pieces * kRowsPerGroup, q_part = 0, q_group = first;
  int q_sub = 0;  // SEQ: 0 the gate row of the group, 1 its up row
  auto q_locate = [&]() {
    if constexpr (SEQ) {
      const uint8_t *pk = q_sub == 0 ? a.packed[0] : a.packed2;
      const uint16_t *sc = q_sub == 0 ? a.scale[0] : a.scale2;
      wq[0] = reinterpret_cast<uint64_t>(pk) + static_cast<uint32_t>(q_group) * row_bytes;
      sq[0] = reinterpret_cast<uint64_t>(sc) + static_cast<uint32_t>(q_group) * row_scale_bytes;
    } else {
      int row = q_group;
      const uint8_t *pk = a.packed[0];
      const uint16_t *sc = a.scale[0];
      if (!one_segment && row >= seg_end0) {
        const bool third = row >= seg_end1;
        pk = third ? a.packed[2] : a.packed[1];
        sc = third ? a.scale[2] : a.scale[1];
        row -= third ? seg_end1 : seg_end0;
      }
      wq[0] = reinterpret_cast<uint64_t>(pk) + static_cast<uint32_t>(row) * row_bytes;
      sq[0] = reinterpret_cast<uint64_t>(sc) + static_cast<uint32_t>(row) * row_scale_bytes;
    }
  };
  // after the last request of a piece
  auto q_advance = [&]() {
    if (--q_left == 0) {
      return;
    }
    if (++q_part < pieces) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        wq[r] += NS * 512;
        sq[r] += NS * 32;
      }
      return;
    }
    q_part = 0;
    if constexpr (SEQ) {
      q_sub ^= 1;
      if (q_sub == 0) {
        q_group += stride;
      }
    } else {
      q_group += stride;
    }
    q_locate();
  };
  if (q_left > 0) {
    q_locate();
  }

  // One half step of one row into its fixed registers: two loads.  The s_nop is for the base
  // registers: where the compiler parks a scalar in a vector register's lane it brings it
  // back with v_readlane, and a vector memory instruction may read a scalar register that a
  // vector instruction wrote only five wait states later.  The compiler inserts those for
  // its own instructions but does not look inside an asm statement (a build that did spill
  // scalars this way sent requests to stale addresses).
#define CHR_RING_LOAD(W, SREG, CLOB, VW, VS, WP, SP, I)                                   \
  asm("s_nop 4\n\t"                                                                       \
      "global_load_dwordx2 " W ", %1, %2 offset:%5 nt\n\t"                                \
      "global_load_ushort " SREG ", %3, %4 offset:%6 nt"                                  \
      : "+s"(tok)                                                                         \
      : "v"(VW), "s"(WP), "v"(VS), "s"(SP), "n"((I) * 512), "n"((I) * 32)                 \
      : CLOB);
  // slot I: half step I of the piece at wq / sq; LASTP = the piece ends its row
#define CHR_RING_REQUEST_FORM(I, VW, VS, OFF) \
  CHR_RING_LOAD(RR1_W(I), RR1_S(I), RR1_CLOB(I), VW, VS, wq[0], sq[0], OFF)
#define CHR_RING_REQUEST(I, LASTP)                                                        \
  if ((I) > kLastReal && (LASTP)) {                                                       \
    CHR_RING_REQUEST_FORM(I, v_w, v_s, 0)                                                 \
  } else if ((I) == kLastReal && ragged && (LASTP)) {                                     \
    CHR_RING_REQUEST_FORM(I, v_wl, v_sl, I)                                               \
  } else {                                                                                \
    CHR_RING_REQUEST_FORM(I, v_w, v_s, I)                                                 \
  }

  // The first NS requests: the first piece of the wavefront's first group (five request
  // instructions and nothing else in the usual case).  A wavefront without work asks for
  // nothing.
  const bool any_work = q_left > 0;
#define CHR_RING_FILL_STEP(I) \
  if constexpr (NS - LAG > (I)) { CHR_RING_REQUEST(I, pieces == 1) }
  // The first kRingEarlySlots slots are requested right after x, the others after the level
  // table has been written: x then queues behind two half steps per wavefront instead of the
  // whole ring (all slots at once: 7168x5120 7.2-7.4 us and 5120x5120 6.1 us against 7.0 and
  // 5.8 us; one early slot is no better than two).
  constexpr int kRingEarlySlots = 2;
#define CHR_RING_FILL_A_STEP(I) \
  if constexpr ((I) < kRingEarlySlots) { CHR_RING_FILL_STEP(I) }
#define CHR_RING_FILL_B_STEP(I) \
  if constexpr ((I) >= kRingEarlySlots) { CHR_RING_FILL_STEP(I) }
#define CHR_RING_FILL_A                                                                   \
  if (any_work) {                                                                         \
    CHR_RING_FILL_A_STEP(0)                                                               \
    CHR_RING_FILL_A_STEP(1)                                                               \
    CHR_RING_FILL_A_STEP(2)                                                               \
    CHR_RING_FILL_A_STEP(3)                                                               \
    CHR_RING_FILL_A_STEP(4)                                                               \
    CHR_RING_FILL_A_STEP(5)                                                               \
    CHR_RING_FILL_A_STEP(6)                                                               \
    CHR_RING_FILL_A_STEP(7)                                                               \
  }
#define CHR_RING_FILL_B                                                                   \
  if (any_work) {                                                                         \
    CHR_RING_FILL_B_STEP(0)                                                               \
    CHR_RING_FILL_B_STEP(1)                                                               \
    CHR_RING_FILL_B_STEP(2)                                                               \
    CHR_RING_FILL_B_STEP(3)                                                               \
    CHR_RING_FILL_B_STEP(4)                                                               \
    CHR_RING_FILL_B_STEP(5)                                                               \
    CHR_RING_FILL_B_STEP(6)                                                               \
    CHR_RING_FILL_B_STEP(7)                                                               \
    if constexpr (LAG == 0) {                                                             \
      q_advance();                                                                        \
    }                                                                                     \
  }
#define CHR_RING_FILL CHR_RING_FILL_A CHR_RING_FILL_B
  // nothing of the compiler's own memory traffic crosses this, nor any statement of the chain
#define CHR_RING_FENCE asm volatile("" : "+s"(tok)::"memory");
  // Order of the first requests: x, then the whole ring of weights, and only then the wait
  // for x: x is the older request, so its (exact) wait does not include the weights, and the
  // memory system works on the first NS half steps of every wavefront while the level table
  // is written and x is staged.
  // x travels in registers that the compiler allocates: between its request and its wait
  // there is only this branch's own straight-line code, nothing that could make the compiler
  // move or spill them (hence the two copies of the ring's fill).
  if (stage_fast_ok(a)) {
    XRegs xr;
    ring_x_request(a, xr, tok);
    CHR_RING_FILL_A
    if constexpr (kRingEarlySlots < NS) { CHR_RING_FENCE }
    fill_level_table<TERMS>(dyn_lds, wave, lane);
    if constexpr (kRingEarlySlots < NS) { CHR_RING_FENCE }
    CHR_RING_FILL_B
    if (!any_work) {
      asm("s_waitcnt vmcnt(0)" : "+s"(tok));
    }
    ring_x_wait<(NS - LAG) * kStepLoads>(xr, tok);
    uint4 xv[kXKeep], xg[kXKeep];
#pragma unroll
    for (int j = 0; j < kXKeep; ++j) {
      xv[j] = make_uint4(xr.v[j].x, xr.v[j].y, xr.v[j].z, xr.v[j].w);
      xg[j] = make_uint4(xr.g[j].x, xr.g[j].y, xr.g[j].z, xr.g[j].w);
    }
    x_store<TERMS == 3>(a, xs, lds, xv, xg, make_uint4(xr.q.x, xr.q.y, xr.q.z, xr.q.w));
  } else {
    // The other staging forms read what they need in loops of their own (loads the compiler
    // counts: its waits then also cover the half steps requested here, which are older).
    CHR_RING_FILL
    fill_level_table<TERMS>(dyn_lds, wave, lane);
    stage_x<TERMS == 3>(a, xs, lds);
  }
#undef CHR_RING_FENCE
#undef CHR_RING_FILL
#undef CHR_RING_FILL_B
#undef CHR_RING_FILL_A
#undef CHR_RING_FILL_B_STEP
#undef CHR_RING_FILL_A_STEP
#undef CHR_RING_FILL_STEP

  float acc[R] = {};
  float sq_acc = 0.f;    // sq_out: sum of squares of what this wavefront has stored
  float gate_sum = 0.f;  // SEQ: the gate row's sum while the up row is walked
  int c_sub = 0;
  auto finish_group = [&](int grp) {
    if constexpr (SEQ) {
      const float sum = wave_sum(acc[0]);
      if (c_sub == 0) {
        gate_sum = sum;
      } else if (lane == 0) {
        a.y[0][grp] = f32_to_bf16(silu(gate_sum) * sum);
      }
    } else {
      int row = grp;
      uint16_t *y = a.y[0];
      const uint16_t *add = a.add[0];
      if (!one_segment && row >= seg_end0) {
        const bool third = row >= seg_end1;
        y = third ? a.y[2] : a.y[1];
        add = third ? a.add[2] : a.add[1];
        row -= third ? seg_end1 : seg_end0;
      }
      float v = wave_sum(acc[0]);
      if (add != nullptr) {
        v += uniform_bf16(add + row);
      }
      const uint16_t stored = f32_to_bf16(v);
      if (lane == 0) {
        y[row] = stored;
      }
      if (a.sq_out != nullptr) {
        const float r = bf16_to_f32(stored);
        sq_acc = fmaf(r, r, sq_acc);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = 0.f;
    }
  };

  // 0 in the lanes that MASK (a scalar lane mask) switches off
#define CHR_RING_MASKED(DST, SRC, MASK) \
  asm("v_cndmask_b32 %0, 0, %1, %2" : "=v"(DST) : "v"(SRC), "s"(MASK))

  // The sums go through the chain of asm statements once per half step, which keeps a half
  // step's products ahead of the next half step's wait: left to itself the compiler sinks
  // all products of a piece to its end and holds every level it has looked up until then.
#define CHR_RING_PIN asm("" : "+v"(acc[0]), "+s"(tok));
  // The half step in slot I, its x pieces X0 / X1: wait for it (WAIT), turn its packed bytes
  // into lookup addresses, which frees the slot's registers, issue this step's request
  // (REQUEST: the slot freed LAG steps ago), and only then look the levels up and multiply: the
  // new request travels while this half step is computed.  MASK_IF says whether the lanes past the row's end are to be
  // switched off.
#define CHR_RING_STEP(I, X0, X1, F, WAIT, REQUEST, MASK_IF, EMPTY_IF)                     \
  if (EMPTY_IF) {                                                                         \
    WAIT                                                                                  \
    REQUEST                                                                               \
  } else {                                                                                \
    const uint4 x0 = X0, x1 = X1;                                                         \
    const uint32_t xw[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};              \
    WAIT                                                                                  \
    {                                                                                     \
      uint32_t aw[8];                                                                     \
      float sw_;                                                                          \
      CHR_RING_ADDRESSES(RR1_X(I), RR1_Y(I), RR1_S(I), aw, sw_, lane_off, tok);           \
      REQUEST                                                                             \
      if (MASK_IF) {                                                                      \
        CHR_RING_MASKED(sw_, sw_, last_lanes);                                            \
      }                                                                                   \
      if constexpr (TERMS == 3) {                                                         \
        sw_ *= F;                                                                         \
      }                                                                                   \
      acc[0] = fmaf(sw_, ring_row_dot<TERMS>(aw, xw), acc[0]);                            \
    }                                                                                     \
    CHR_RING_PIN                                                                          \
  }

  // steady state: D-1-LAG younger half steps are in flight when a step waits for its own
#define CHR_RING_WAIT_FULL(I) \
  asm("s_waitcnt vmcnt(%1)" : "+s"(tok) : "n"((D - 1 - LAG) * kStepLoads));
  // the last piece requests only its own last LAG slots (in its first LAG steps): step I has
  // D-1-I younger half steps behind it at most
#define CHR_RING_WAIT_LAST(I)              \
  asm("s_waitcnt vmcnt(%1)" : "+s"(tok) \
      : "n"(((D - 1 - (I)) < (D - 1 - LAG) ? (D - 1 - (I)) : (D - 1 - LAG)) * kStepLoads));

  // ---- the groups, a piece per turn --------------------------------------------------------
  int c_left = my_groups * pieces * kRowsPerGroup, c_part = 0, c_group = first;
  // XREG (a row is one piece of at most 5 half steps): the lane's x pieces of the whole row
  // stay in registers, which takes two 16-byte LDS reads out of every half step.
  uint4 x_row[XREG ? 2 * NS : 1];
  float f_row[XREG && TERMS == 3 ? NS : 1];
  if constexpr (XREG) {
    if (c_left > 0) {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        x_row[2 * i] = lds0_u128(x_lane + i * 2048);
        x_row[2 * i + 1] = lds0_u128(x_lane + i * 2048 + 1024);
        if constexpr (TERMS == 3) {
          f_row[i] = lds0_at(f_lane + i * 256);
        }
      }
    }
  }
#define CHR_RING_OWN_STEP(I, WAIT, REQUEST)                                               \
  if constexpr (NS > (I)) {                                                               \
    if constexpr (XREG) {                                                                 \
      CHR_RING_STEP(I, x_row[2 * ((I) % NS)], x_row[2 * ((I) % NS) + 1],                  \
                    f_row[TERMS == 3 ? (I) % NS : 0], WAIT, REQUEST,                      \
                    (I) == NS - 1 && ragged, false)                                       \
    } else {                                                                              \
      CHR_RING_STEP(I, lds0_u128(xa + (I) * 2048), lds0_u128(xa + (I) * 2048 + 1024),     \
                    lds0_at(fa + (I) * 256), WAIT,                                        \
                    REQUEST, (I) == kLastReal && ragged && c_last, (I) > kLastReal && c_last) \
    }                                                                                     \
  }
#define CHR_RING_PIECE(WAIT_OF, REQUEST_OF)                                               \
  {                                                                                       \
    const uint32_t xa = x_lane + static_cast<uint32_t>(c_part) * (NS * 2048);             \
    const uint32_t fa = f_lane + static_cast<uint32_t>(c_part) * (NS * 256);              \
    const bool c_last = c_part == pieces - 1;                                             \
    CHR_RING_OWN_STEP(0, WAIT_OF(0), REQUEST_OF(0))                                       \
    CHR_RING_OWN_STEP(1, WAIT_OF(1), REQUEST_OF(1))                                       \
    CHR_RING_OWN_STEP(2, WAIT_OF(2), REQUEST_OF(2))                                       \
    CHR_RING_OWN_STEP(3, WAIT_OF(3), REQUEST_OF(3))                                       \
    CHR_RING_OWN_STEP(4, WAIT_OF(4), REQUEST_OF(4))                                       \
    CHR_RING_OWN_STEP(5, WAIT_OF(5), REQUEST_OF(5))                                       \
    CHR_RING_OWN_STEP(6, WAIT_OF(6), REQUEST_OF(6))                                       \
    CHR_RING_OWN_STEP(7, WAIT_OF(7), REQUEST_OF(7))                                       \
    --c_left;                                                                             \
    if (c_last) {                                                                         \
      finish_group(c_group);                                                              \
      if constexpr (SEQ) {                                                                \
        c_sub ^= 1;                                                                       \
        if (c_sub == 0) {                                                                 \
          c_group += stride;                                                              \
        }                                                                                 \
      } else {                                                                            \
        c_group += stride;                                                                \
      }                                                                                   \
      c_part = 0;                                                                         \
    } else {                                                                              \
      ++c_part;                                                                           \
    }                                                                                     \
    (void)xa;                                                                             \
    (void)fa;                                                                             \
  }
  // slot S (a constant expression) of the piece at the request cursor; the cursor moves on
  // with the piece's last slot
#define CHR_RING_REQUEST_SLOT(S)                                                          \
  {                                                                                       \
    const bool lastp = q_part == pieces - 1;                                              \
    if constexpr ((S) == 0) { CHR_RING_REQUEST(0, lastp) }                                \
    if constexpr ((S) == 1) { CHR_RING_REQUEST(1, lastp) }                                \
    if constexpr ((S) == 2) { CHR_RING_REQUEST(2, lastp) }                                \
    if constexpr ((S) == 3) { CHR_RING_REQUEST(3, lastp) }                                \
    if constexpr ((S) == 4) { CHR_RING_REQUEST(4, lastp) }                                \
    if constexpr ((S) == 5) { CHR_RING_REQUEST(5, lastp) }                                \
    if constexpr ((S) == 6) { CHR_RING_REQUEST(6, lastp) }                                \
    if constexpr ((S) == 7) { CHR_RING_REQUEST(7, lastp) }                                \
    if constexpr ((S) == NS - 1) { q_advance(); }                                         \
  }
  // step I asks again for the slot that step I - LAG consumed
#define CHR_RING_REQUEST_NEXT(I) CHR_RING_REQUEST_SLOT(((I) + NS - LAG) % NS)
  // the last piece: its own last LAG slots, then nothing
#define CHR_RING_REQUEST_LAST(I) \
  if constexpr ((I) < LAG) { CHR_RING_REQUEST_SLOT(NS - LAG + (I)) }
  // while a piece after the one being computed is left to request
  while (q_left > (LAG > 0 ? 1 : 0)) {
    CHR_RING_PIECE(CHR_RING_WAIT_FULL, CHR_RING_REQUEST_NEXT)
  }
  // the last piece
  if (c_left > 0) {
    CHR_RING_PIECE(CHR_RING_WAIT_LAST, CHR_RING_REQUEST_LAST)
  }
  // nothing may still be on its way into the fixed registers when the wavefront ends (this
  // statement is volatile: it is what keeps the token chain, and with it every request, alive)
  asm volatile("s_waitcnt vmcnt(0)" : "+s"(tok));
  if constexpr (!SEQ) {
    if (a.sq_out != nullptr) {
      store_sumsq_part(a, lds, sq_acc, wave, lane);
    }
  }
#undef CHR_RING_REQUEST_LAST
#undef CHR_RING_REQUEST_NEXT
#undef CHR_RING_REQUEST_SLOT
#undef CHR_RING_PIECE
#undef CHR_RING_OWN_STEP
#undef CHR_RING_WAIT_LAST
#undef CHR_RING_WAIT_FULL
#undef CHR_RING_STEP
#undef CHR_RING_PIN
#undef CHR_RING_MASKED
#undef CHR_RING_REQUEST
#undef CHR_RING_REQUEST_FORM
#undef CHR_RING_LOAD
}

// The compiler's VGPR budget stops where the ring's fixed registers begin.  (On this target
// the attribute counts vector and accumulation registers together and is ignored when the
// sum exceeds what the launch bounds allow, so it names half the vector registers meant.)
template <int NS, int TERMS, bool XREG, int PAD = 0, bool SEQ = false>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_num_vgpr(52))) void gemv_ring_rows(
    const StreamArgs a) {
  gemv_ring_body<NS, TERMS, XREG, PAD, SEQ>(a);
}

// Half steps of a piece (= slots of the ring, 544 bytes per row each) for a row of nsteps
// half steps: the largest divisor in 7..4, so that 2 to 4 KB per wavefront are in flight (a
// pure streaming read of a 35 MB matrix by this grid is fastest with 2 KB per wavefront on the
// way and loses 15% at 4 KB; eight slots, 4.3 KB, measured 9.36 against 8.92 us with four at
// 8192x8192 and 11.73 against 11.56 at 6144x16384, while six beat four at 5120x12288, 8.5
// against 8.7).  A row kernel also takes a length one half step short of a multiple of 5..8
// (11 = 2 * 6 - 1, 27 = 4 * 7 - 1), its last piece ending in one empty slot.  steps == 0: the
// ring kernel does not take this row length (the compiler-pipelined kernel does).
struct RingPiece {
  int steps;
  int pad;
};
RingPiece ring_piece_steps(int nsteps) {
  for (int ns = 7; ns >= 4; --ns) {
    if (nsteps % ns == 0) {
      return {ns, 0};
    }
  }
  if (nsteps > 8) {
    for (const int ns : {7, 6, 5, 8}) {
      if ((nsteps + 1) % ns == 0) {
        return {ns, 1};
      }
    }
  }
  return {0, 0};
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

// Form of the levels in the kernels that stage x in LDS (CHR_NF4_GEMV_TERMS, read on every
// launch): 3 = one binary16 against x staged as binary16 (2^-12 relative weight error; "3" or
// "f16"), 2 = head + tail bf16 (below 2^-17; "2"), 1 = one bf16 (2^-9; "1").
#ifndef CHR_NF4_DEFAULT_TERMS
#define CHR_NF4_DEFAULT_TERMS 3
#endif
int level_terms() {
  const char *e = std::getenv("CHR_NF4_GEMV_TERMS");
  if (e != nullptr && e[0] != '\0') {
    if (e[0] == '1' && e[1] == '\0') {
      return 1;
    }
    if (e[0] == '2' && e[1] == '\0') {
      return 2;
    }
    if ((e[0] == '3' && e[1] == '\0') || (e[0] == 'f' && e[1] == '1' && e[2] == '6' && e[3] == '\0')) {
      return 3;
    }
  }
  return CHR_NF4_DEFAULT_TERMS;
}

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

// Half steps per item of the staged kernel.  Measured on the 14B shapes: one step leaves
// too little in flight (13824x5120: 12.9 us), two are best (10.3 us), three and five cost
// more again (10.4, 11.0 us) -- deeper request queues do not pay on this memory system.
constexpr int kItemSteps = 2;

// pair table, small statics, x pieces, the binary16 form's inverse powers (a float per lane and half step)
inline size_t staged_lds_bytes(int K_pad) {
  return kPairTableBytes + kStagedSmallBytes + static_cast<size_t>(x_pieces(K_pad)) * 16 +
         static_cast<size_t>(x_half_steps(K_pad)) * kWave * sizeof(float);
}

// Whether staged launches go to the ring kernels where those take the row length: yes.
// Measured, one-term / two-term levels, ring against pipelined (us): 13824x5120 9.7 / 10.6
// against 10.8 / 11.6; 5120x13824 10.1 / 10.7 against 11.3 / 11.2; 27648x5120 16.4 / 18.1
// against 18.6 / 20.7; 152064x5120 72 / 80 against 77 / 89; gate/up 13824x5120 17.3 / 19.4
// against 20.0 / 21.6; 7168x5120, 5120x5120 and 4096x4096 within 3% either way.
// CHR_NF4_GEMV_RING=0 keeps every staged launch on the compiler-pipelined kernel (read on
// every launch).
bool ring_wanted() {
  const char *e = std::getenv("CHR_NF4_GEMV_RING");
  return !(e != nullptr && e[0] == '0' && e[1] == '\0');
}

// Kernel family for a launch of m_total weight rows: 1 staged, 0 plain, -1 staging is
// required but x does not fit the LDS.  Staging is required by the fused RMSNorm, a
// ragged K and the attention merge; otherwise the staged kernel is taken from 16M codes
// up (below that its set-up costs more than its cheaper inner loop returns: 2048x2048
// measures 4.2 us staged, 3.9 us plain; 11008x2048 6.0 against 6.2 us).
int pick_family(const StreamArgs &a, int m_total) {
  const bool fits = staged_lds_bytes(a.K_pad) <= kMaxDynLds;
  if (a.rms_w != nullptr || a.K != a.K_pad || a.attn_state != nullptr) {
    return fits ? 1 : -1;
  }
  const int forced = forced_staged();
  if (forced >= 0) {
    return forced == 1 && fits ? 1 : 0;
  }
  const long long codes = static_cast<long long>(m_total) * a.K_pad;
  return fits && codes >= (16ll << 20) ? 1 : 0;
}

// Rows per wavefront of the staged kernels: one, so that even 5120 rows give every
// wavefront of 256 compute units work; the ring kernel (one row) where ring_wanted says so
// and it takes the row length; else two rows from 32768 up (lm_head 152064x5120: 75 us
// against 81 us).
int staged_rows_for_m(int M, int K_pad) {
  const int f = forced_rows();
  if (f > 0) {
    return f;
  }
  if (ring_wanted() && ring_piece_steps(x_half_steps(K_pad)).steps > 0) {
    return 1;  // the ring kernel walks one row (or one gate/up pair) per group
  }
  return M >= 32768 ? 2 : 1;
}

// Whether a launch can take its mean(x^2) from parts a writer left: the staging that keeps x in
// registers between its request and its use (the device's stage_fast_ok), on a staged kernel.
bool sumsq_in_ok(const StreamArgs &a, bool staged) {
  return staged && a.rms_w != nullptr && a.attn_state == nullptr && (a.K & 7) == 0 &&
         aligned16(a.x) && aligned16(a.rms_w) && aligned16(a.sq_in) &&
         (a.K_pad >> 3) <= kXKeep * kStagedThreads;
}

template <int R, bool SWIGLU>
int launch_stream(StreamArgs &a, int n_seg, bool staged, hipStream_t st) {
  constexpr int U = SWIGLU ? R / 2 : R;
  if (a.sq_in != nullptr && !sumsq_in_ok(a, staged)) {
    return -8;
  }
  if (a.sq_out != nullptr && (!staged || SWIGLU || n_seg != 1 ||
                              (reinterpret_cast<uintptr_t>(a.sq_out) & 3u) != 0)) {
    return -8;  // the staged kernels of a single matrix write the parts
  }
  int total = 0;
  for (int i = 0; i < 3; ++i) {
    a.groups[i] = i < n_seg ? (a.M[i] + U - 1) / U : 0;
    total += a.groups[i];
  }
  if (staged) {
    const size_t dyn = staged_lds_bytes(a.K_pad);
    const int waves = kStagedThreads / kWave;
    const int grid = std::min(device_cu_count(), (total + waves - 1) / waves);
    const int terms = level_terms();
    constexpr bool kRingShape = (SWIGLU && R == 2) || (!SWIGLU && R == 1);  // one row, or one gate/up pair, a group
    const RingPiece ring = kRingShape && ring_wanted()
                               ? ring_piece_steps(x_half_steps(a.K_pad)) : RingPiece{0, 0};
    const int ring_ns = ring.steps;
    // wavefront w of workgroup b walks groups w * grid + b, + 16 * grid, ..: full passes, and one
    // more for the first ring_left wavefronts
    const int per_pass = grid * waves;
    a.ring_grid = grid;
    a.ring_passes = total / per_pass;
    a.ring_left = total % per_pass;
    if (a.sq_out != nullptr && grid > kSumsqParts) {
      return -8;
    }
    if (ring_ns > 0) {
      if constexpr (kRingShape) {
        auto go = [&](auto kern) {
          if (prep_lds(kern, dyn) != 0) {
            return -6;
          }
          kern<<<dim3(grid), dim3(kStagedThreads), dyn, st>>>(a);
          return 0;
        };
        int rc = -6;
        // a row that is one piece of at most 5 half steps keeps its x in registers
        const bool one_piece = x_half_steps(a.K_pad) == ring_ns && ring_ns <= 5;
        // the kernel for NS slots by the form of the levels
#define CHR_GO_ROWS(NS, XREG, PAD)                                                        \
  (terms == 1 ? go(gemv_ring_rows<NS, 1, XREG, PAD>)                                      \
   : terms == 3 ? go(gemv_ring_rows<NS, 3, XREG, PAD>) : go(gemv_ring_rows<NS, 2, XREG, PAD>))
#define CHR_GO_SEQ(NS, XREG, PAD)                                                         \
  (terms == 1 ? go(gemv_ring_rows<NS, 1, XREG, PAD, true>)                                \
   : terms == 3 ? go(gemv_ring_rows<NS, 3, XREG, PAD, true>) : go(gemv_ring_rows<NS, 2, XREG, PAD, true>))
        if constexpr (SWIGLU) {
          // gate row, then up row of the same index, through the single-row ring
          switch (ring.pad > 0 ? -ring_ns : ring_ns) {
            case -5: rc = CHR_GO_SEQ(5, false, 1); break;
            case -6: rc = CHR_GO_SEQ(6, false, 1); break;
            case -7: rc = CHR_GO_SEQ(7, false, 1); break;
            case -8: rc = CHR_GO_SEQ(8, false, 1); break;
            case 4: rc = one_piece ? CHR_GO_SEQ(4, true, 0) : CHR_GO_SEQ(4, false, 0); break;
            case 5: rc = one_piece ? CHR_GO_SEQ(5, true, 0) : CHR_GO_SEQ(5, false, 0); break;
            case 6: rc = CHR_GO_SEQ(6, false, 0); break;
            case 7: rc = CHR_GO_SEQ(7, false, 0); break;
          }
        } else {
          switch (ring.pad > 0 ? -ring_ns : ring_ns) {
            case -5: rc = CHR_GO_ROWS(5, false, 1); break;
            case -6: rc = CHR_GO_ROWS(6, false, 1); break;
            case -7: rc = CHR_GO_ROWS(7, false, 1); break;
            case -8: rc = CHR_GO_ROWS(8, false, 1); break;
            case 4: rc = one_piece ? CHR_GO_ROWS(4, true, 0) : CHR_GO_ROWS(4, false, 0); break;
            case 5: rc = one_piece ? CHR_GO_ROWS(5, true, 0) : CHR_GO_ROWS(5, false, 0); break;
            case 6: rc = CHR_GO_ROWS(6, false, 0); break;
            case 7: rc = CHR_GO_ROWS(7, false, 0); break;
          }
        }
#undef CHR_GO_SEQ
#undef CHR_GO_ROWS
        if (rc != 0) {
          return rc;
        }
      }
    } else if (terms == 1) {
      constexpr auto kern = gemv_staged<R, kItemSteps, SWIGLU, 1>;
      if (prep_lds(kern, dyn) != 0) {
        return -6;
      }
      kern<<<dim3(grid), dim3(kStagedThreads), dyn, st>>>(a);
    } else if (terms == 3) {
      constexpr auto kern = gemv_staged<R, kItemSteps, SWIGLU, 3>;
      if (prep_lds(kern, dyn) != 0) {
        return -6;
      }
      kern<<<dim3(grid), dim3(kStagedThreads), dyn, st>>>(a);
    } else {
      constexpr auto kern = gemv_staged<R, kItemSteps, SWIGLU, 2>;
      if (prep_lds(kern, dyn) != 0) {
        return -6;
      }
      kern<<<dim3(grid), dim3(kStagedThreads), dyn, st>>>(a);
    }
  } else {
    const int waves = kThreads / kWave;
    // Long rows and few of them (a down projection): a wavefront walking a whole row pays
    // the memory latency once per step, so the four wavefronts of a workgroup split the
    // steps of one row group instead.
    const int nsteps = (a.K_pad + 2047) / 2048;
    const bool split = !SWIGLU && nsteps >= 4 && total * 4 <= 16 * device_cu_count() * 4;
    a.ksplit = split ? waves : 1;
    const int grid = split ? total : (total + waves - 1) / waves;
    gemv_stream<R, SWIGLU><<<dim3(grid), dim3(kThreads), 0, st>>>(a);
  }
  return launch_rc();
}

int launch_rows(StreamArgs &a, int n_seg, int m_for_policy, hipStream_t st) {
  const int family = pick_family(a, m_for_policy);
  if (family < 0) {
    return -6;
  }
  const bool staged = family == 1;
  switch (staged ? staged_rows_for_m(m_for_policy, a.K_pad) : rows_for_m(m_for_policy)) {
    case 4:
      return launch_stream<4, false>(a, n_seg, staged, st);
    case 2:
      return launch_stream<2, false>(a, n_seg, staged, st);
    default:
      return launch_stream<1, false>(a, n_seg, staged, st);
  }
}

// A gate/up pair is two weight streams per output row: the staged kernel takes one pair
// per wavefront (two from 32768 pairs up), the plain one two pairs when there are enough.
int launch_pairs(StreamArgs &a, int m_pairs, hipStream_t st) {
  const int family = pick_family(a, 2 * m_pairs);
  if (family < 0) {
    return -6;
  }
  const bool staged = family == 1;
  const int rows = staged ? 2 * staged_rows_for_m(m_pairs, a.K_pad) : (rows_for_m(2 * m_pairs) >= 2 ? 4 : 2);
  if (rows >= 4) {
    return launch_stream<4, true>(a, 1, staged, st);
  }
  return launch_stream<2, true>(a, 1, staged, st);
}

}  // namespace

// Shared with the GEMM entry points, which route N == 1 here.
int gemv_entry(const chr_nf4_dev_t *w, const void *x, void *y, void *stream, const void *add,
               const void *rms_w, float rms_eps, const float *sq_in, float *sq_out) {
  if (w == nullptr || x == nullptr || y == nullptr) {
    return -1;
  }
  if (sq_in != nullptr && rms_w == nullptr) {
    return -8;
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
  a.sq_in = sq_in;
  a.sq_out = sq_out;
  return launch_rows(a, 1, w->M, static_cast<hipStream_t>(stream));
}

// y = W @ merge(states) (+ add): the o projection consuming what chr_dv2_attn_parts left.
int gemv_attn_entry(const chr_nf4_dev_t *w, const float *state, int n_q, int hd, int n_parts,
                    void *y, const void *add, void *stream, float *sq_out) {
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
  a.sq_out = sq_out;
  return launch_rows(a, 1, w->M, static_cast<hipStream_t>(stream));
}

// Whether a single-matrix GEMV of this shape (merging attention states or not) runs on the
// kernel that can leave the sum of squares of its output (chr_dv2_sumsq_ok).
bool gemv_sumsq_out_ok(int M, int K, int K_pad, bool merges_attention) {
  if (M < 1 || K < 1 || !k_pad_ok(K, K_pad)) {
    return false;
  }
  StreamArgs a{};
  a.K = K;
  a.K_pad = K_pad;
  if (merges_attention) {
    a.attn_state = reinterpret_cast<const float *>(&a);  // only tested against nullptr
  }
  if (pick_family(a, M) != 1) {
    return false;
  }
  const int waves = kStagedThreads / kWave;
  const int groups = (M + staged_rows_for_m(M, K_pad) - 1) / staged_rows_for_m(M, K_pad);
  return std::min(device_cu_count(), (groups + waves - 1) / waves) <= kSumsqParts;
}

// Launch geometry of the N=1 path, reported by the planner: what chr_nf4_gemv launches for
// this matrix without fused extras.
bool gemv_plan_staged(int M, int K, int K_pad) {
  StreamArgs a{};
  a.K = K;
  a.K_pad = K_pad;
  return pick_family(a, M) == 1;
}

int gemv_rows_per_wg(int M, int K, int K_pad) {
  return gemv_plan_staged(M, K, K_pad) ? (kStagedThreads / kWave) * staged_rows_for_m(M, K_pad)
                                       : (kThreads / kWave) * rows_for_m(M);
}

int gemv_threads_per_wg(int M, int K, int K_pad) {
  return gemv_plan_staged(M, K, K_pad) ? kStagedThreads : kThreads;
}

int gemv_grid_x(int M, int K, int K_pad) {
  const int bm = gemv_rows_per_wg(M, K, K_pad);
  const int blocks = (M + bm - 1) / bm;
  return gemv_plan_staged(M, K, K_pad) ? std::min(device_cu_count(), blocks) : blocks;
}

// codes of a row one wavefront request covers
int gemv_step_codes(int M, int K, int K_pad) { return gemv_plan_staged(M, K, K_pad) ? 1024 : 2048; }

int gemv_lds_bytes(int M, int K, int K_pad) {
  return gemv_plan_staged(M, K, K_pad) ? static_cast<int>(staged_lds_bytes(K_pad))
                                       : static_cast<int>(sizeof(GemvLds));
}

}  // namespace chr

using namespace chr;

extern "C" int chr_nf4_gemv(const chr_nf4_dev_t *w, const void *x, void *y, void *stream,
                            const void *add, const void *rms_w, float rms_eps) {
  return gemv_entry(w, x, y, stream, add, rms_w, rms_eps, nullptr, nullptr);
}

extern "C" int chr_dv2_gemv_sumsq(const chr_nf4_dev_t *w, const void *x, void *y, void *stream,
                                  const void *add, const void *rms_w, float rms_eps,
                                  const float *sumsq_in, float *sumsq_out) {
  return gemv_entry(w, x, y, stream, add, rms_w, rms_eps, sumsq_in, sumsq_out);
}

extern "C" int32_t chr_dv2_sumsq_parts(void) { return kSumsqParts; }

extern "C" int32_t chr_dv2_sumsq_ok(int32_t M, int32_t K, int32_t K_pad, int32_t merges_attention) {
  return gemv_sumsq_out_ok(M, K, K_pad, merges_attention != 0) ? 1 : 0;
}

namespace chr {
namespace {
int qkv_entry(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k, const chr_nf4_dev_t *v, const void *x,
              void *yq, void *yk, void *yv, const void *bq, const void *bk, const void *bv,
              void *stream, const void *rms_w, float rms_eps, const float *sq_in) {
  if (sq_in != nullptr && rms_w == nullptr) {
    return -8;
  }
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
  a.sq_in = sq_in;
  return launch_rows(a, 3, q->M + k->M + v->M, static_cast<hipStream_t>(stream));
}

int swiglu_entry(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up, const void *x, void *y,
                 void *stream, const void *rms_w, float rms_eps, const float *sq_in) {
  if (sq_in != nullptr && rms_w == nullptr) {
    return -8;
  }
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
  a.sq_in = sq_in;
  return launch_pairs(a, gate->M, static_cast<hipStream_t>(stream));
}
}  // namespace
}  // namespace chr

extern "C" int chr_nf4_gemv_qkv(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                                const chr_nf4_dev_t *v, const void *x, void *yq, void *yk,
                                void *yv, const void *bq, const void *bk, const void *bv,
                                void *stream, const void *rms_w, float rms_eps) {
  return qkv_entry(q, k, v, x, yq, yk, yv, bq, bk, bv, stream, rms_w, rms_eps, nullptr);
}

extern "C" int chr_dv2_gemv_qkv_sumsq(const chr_nf4_dev_t *q, const chr_nf4_dev_t *k,
                                      const chr_nf4_dev_t *v, const void *x, void *yq, void *yk,
                                      void *yv, const void *bq, const void *bk, const void *bv,
                                      void *stream, const void *rms_w, float rms_eps,
                                      const float *sumsq_in) {
  return qkv_entry(q, k, v, x, yq, yk, yv, bq, bk, bv, stream, rms_w, rms_eps, sumsq_in);
}

extern "C" int chr_nf4_gemv_swiglu(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                                   const void *x, void *y, void *stream, const void *rms_w,
                                   float rms_eps) {
  return swiglu_entry(gate, up, x, y, stream, rms_w, rms_eps, nullptr);
}

extern "C" int chr_dv2_gemv_swiglu_sumsq(const chr_nf4_dev_t *gate, const chr_nf4_dev_t *up,
                                         const void *x, void *y, void *stream, const void *rms_w,
                                         float rms_eps, const float *sumsq_in) {
  return swiglu_entry(gate, up, x, y, stream, rms_w, rms_eps, sumsq_in);
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

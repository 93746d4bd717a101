// Shared device helpers for the gfx950 NF4 kernels: the 16-level codebook,
// bf16 / binary16 bit conversions, and 64-lane wavefront reductions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/chr_nf4_amd.h"

namespace chr {

constexpr int kGroup = 64;  // weights per scale
constexpr int kWave = 64;   // lanes per wavefront on gfx950
// Floats of a sum of squares handed from the launch that writes a vector to the launch that
// normalises it (one part per workgroup of the writer, zeros behind them; a lane of the reader
// takes four).
constexpr int kSumsqParts = 256;

// binary32 bit patterns of the QLoRA NF4 levels (internal/nf4/nf4.go:18-35,
// bits as listed in internal/nf4/nf4_test.go:12-29).
#define CHR_NF4_LEVEL_BITS                                                                   \
  0xBF800000u, 0xBF3239B1u, 0xBF066B30u, 0xBECA32A0u, 0xBE91A24Du, 0xBE3D353Fu, 0xBDBA7871u, \
      0x00000000u, 0x3DA2FAFFu, 0x3E24CAE3u, 0x3E7C04DDu, 0x3EAD033Au, 0x3EE1A4B8u,          \
      0x3F1007ABu, 0x3F3913B3u, 0x3F800000u
__device__ __constant__ const uint32_t kLutBits[16] = {CHR_NF4_LEVEL_BITS};
// the same sixteen words for code that wants them as compile-time constants
constexpr uint32_t kLevelBits[16] = {CHR_NF4_LEVEL_BITS};

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __float_as_uint(f); }

// bf16 bits -> f32: the 16 bits are the top half of the binary32 word.
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return bits_to_f32(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return bits_to_f32(pair & 0xFFFF0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return bits_to_f32(static_cast<uint32_t>(h) << 16);
}

// f32 -> bf16 bits, round to nearest even, NaN stays NaN: the conversion instruction of gfx950
// (v_cvt_pk_bf16_f32), which rounds every finite value as the closed form of
// internal/f16/f16.go:93-106 does.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

// two values in one instruction: lo in bits 0..15, hi in bits 16..31
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float F32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 Bf16x2Bits;
  const F32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, Bf16x2Bits));
}

// binary16 bits -> f32, exact (v_cvt_f32_f16 widens subnormals exactly).
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}

// f32 -> binary16 bits, round to nearest even, written out in integer
// arithmetic so it matches internal/f16/f16.go:8-57 case for case.
__device__ __forceinline__ uint16_t f32_to_f16_rne(float f) {
  const uint32_t b = f32_to_bits(f);
  const uint32_t sign = (b >> 16) & 0x8000u;
  const int exp = static_cast<int>((b >> 23) & 0xFFu);
  uint32_t man = b & 0x7FFFFFu;
  if (exp == 0xFF) {
    if (man != 0) {
      uint32_t n = man >> 13;
      if (n == 0) {
        n = 1;
      }
      return static_cast<uint16_t>(sign | 0x7C00u | n);
    }
    return static_cast<uint16_t>(sign | 0x7C00u);
  }
  const int e = exp - 127 + 15;
  if (e >= 0x1F) {
    return static_cast<uint16_t>(sign | 0x7C00u);
  }
  if (e <= 0) {
    if (e < -10) {
      return static_cast<uint16_t>(sign);
    }
    man |= 1u << 23;
    const uint32_t shift = static_cast<uint32_t>(14 - e);
    const uint32_t round = (man >> (shift - 1)) & 1u;
    const uint32_t tail = man & ((1u << (shift - 1)) - 1u);
    uint32_t m = man >> shift;
    if (round != 0 && (tail != 0 || (m & 1u) != 0)) {
      ++m;
    }
    return static_cast<uint16_t>(sign | m);
  }
  uint32_t half = sign | (static_cast<uint32_t>(e) << 10) | (man >> 13);
  const uint32_t rem = man & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u) != 0)) {
    ++half;
  }
  return static_cast<uint16_t>(half);
}

// ---- cross-lane helpers ------------------------------------------------------
// DPP controls (row = 16 lanes).
constexpr int kDppQuadXor1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppRowMirror = 0x140;     // lane i <-> 15-i inside each 16

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
  return __int_as_float(r);
}

// Sum over aligned groups of LANES lanes (a power of two); every lane of the
// group ends with the group's sum.  Up to 16 lanes this is pure DPP.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16 ||
                    LANES == 32 || LANES == 64,
                "group size must be a power of two up to 64");
  if constexpr (LANES >= 2) v += dpp_f32<kDppQuadXor1>(v);
  if constexpr (LANES >= 4) v += dpp_f32<kDppQuadXor2>(v);
  if constexpr (LANES >= 8) v += dpp_f32<kDppRowHalfMirror>(v);
  if constexpr (LANES >= 16) v += dpp_f32<kDppRowMirror>(v);
  if constexpr (LANES >= 32) v += __shfl_xor(v, 16, kWave);
  if constexpr (LANES >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

template <int LANES>
__device__ __forceinline__ float group_max(float v) {
  if constexpr (LANES >= 2) v = fmaxf(v, dpp_f32<kDppQuadXor1>(v));
  if constexpr (LANES >= 4) v = fmaxf(v, dpp_f32<kDppQuadXor2>(v));
  if constexpr (LANES >= 8) v = fmaxf(v, dpp_f32<kDppRowHalfMirror>(v));
  if constexpr (LANES >= 16) v = fmaxf(v, dpp_f32<kDppRowMirror>(v));
  if constexpr (LANES >= 32) v = fmaxf(v, __shfl_xor(v, 16, kWave));
  if constexpr (LANES >= 64) v = fmaxf(v, __shfl_xor(v, 32, kWave));
  return v;
}

// Whole-wavefront sum, result uniform in every lane: four DPP steps fold each
// row of 16, then the four row totals are read as scalars and added in a fixed
// order (deterministic, no atomics).
__device__ __forceinline__ float wave_sum(float v) {
  v = group_sum<16>(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (r0 + r1) + (r2 + r3);
}

// ---- streaming loads -------------------------------------------------------------
// Packed weights and their scales are read once per launch: the non-temporal hint (the nt bit
// of the load) keeps them from displacing what is reused (x, tables, the KV cache) on their
// way through the caches.  Measured on the N=1 kernel: 11.1 -> 10.1 us at 13824x5120.
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint4 stream_load16(const void *p) {
  const U32x4 v = __builtin_nontemporal_load(static_cast<const U32x4 *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ uint2 stream_load8(const void *p) {
  const U32x2 v = __builtin_nontemporal_load(static_cast<const U32x2 *>(p));
  return make_uint2(v.x, v.y);
}

__device__ __forceinline__ uint16_t stream_load2(const uint16_t *p) {
  return __builtin_nontemporal_load(p);
}

// ---- host-side argument checks shared by the entry points -------------------
inline bool k_pad_ok(int K, int K_pad) {
  if (K < 1 || K_pad < K) {
    return false;
  }
  return K_pad == kGroup * ((K + kGroup - 1) / kGroup);
}

__host__ __device__ inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__host__ __device__ inline bool aligned2(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

// ---- codebook lookups shared by the GEMV and GEMM kernels -------------------------
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

// Eight codes of one dword -> eight codebook levels.  In (w << 2) byte j
// carries 4*code(2j) in bits 2..5; in (w >> 2) byte j carries 4*code(2j+1)
// there.  Masking a selected byte with 0x3C is the LDS byte offset of the level.
struct Levels8 {
  float l[8];
};

__device__ __forceinline__ Levels8 lookup8(uint32_t w, const float *lut) {
  const uint32_t ev = w << 2;
  const uint32_t od = w >> 2;
  const uint32_t mask = 0x3Cu;
  Levels8 r;
  r.l[0] = lut_at(lut, and_byte<0>(ev, mask));
  r.l[1] = lut_at(lut, and_byte<0>(od, mask));
  r.l[2] = lut_at(lut, and_byte<1>(ev, mask));
  r.l[3] = lut_at(lut, and_byte<1>(od, mask));
  r.l[4] = lut_at(lut, and_byte<2>(ev, mask));
  r.l[5] = lut_at(lut, and_byte<2>(od, mask));
  r.l[6] = lut_at(lut, and_byte<3>(ev, mask));
  r.l[7] = lut_at(lut, and_byte<3>(od, mask));
  return r;
}

// lookup8 for a kernel whose 16 levels sit at LDS address 0 and whose LDS is all dynamic
// (the compiler then does not know the base and would add it to every offset): the byte
// offset is the whole address.
__device__ __forceinline__ float lds0_at(uint32_t off) {
  return *reinterpret_cast<const __attribute__((address_space(3))) float *>(off);
}

__device__ __forceinline__ Levels8 lookup8_lds0(uint32_t w) {
  const uint32_t ev = w << 2;
  const uint32_t od = w >> 2;
  const uint32_t mask = 0x3Cu;
  Levels8 r;
  r.l[0] = lds0_at(and_byte<0>(ev, mask));
  r.l[1] = lds0_at(and_byte<0>(od, mask));
  r.l[2] = lds0_at(and_byte<1>(ev, mask));
  r.l[3] = lds0_at(and_byte<1>(od, mask));
  r.l[4] = lds0_at(and_byte<2>(ev, mask));
  r.l[5] = lds0_at(and_byte<2>(od, mask));
  r.l[6] = lds0_at(and_byte<3>(ev, mask));
  r.l[7] = lds0_at(and_byte<3>(od, mask));
  return r;
}

// ---- pair table (kernels that stage x in LDS) ---------------------------------------
// One packed byte holds two codes; the table maps a byte to the two levels as a bf16
// pair, and every lane owns a copy: entry (byte, lane) is the dword at byte address
// byte*256 + lane*4, so the 64 lookups of a wavefront always fall in 64 different banks
// whatever the codes are.  The table starts at LDS address 0 (these kernels have no
// static LDS), which makes a lookup address one v_perm_b32: byte 1 = the packed byte,
// byte 0 = 4*lane.  A pair meets two activations, kept as the bf16 pair they arrive as,
// in one v_dot2c_f32_bf16, or sits as two elements of a matrix-core operand: per two
// weights one address op and one LDS read, against two of each with the 16-entry table.
constexpr int kPairTableBytes = 256 * 64 * 4;

__device__ __forceinline__ uint32_t lds0_u32(uint32_t addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>(addr);
}

template <int J>
__device__ __forceinline__ uint32_t pair_at(uint32_t w, uint32_t lane4) {
  // selector: result byte 0 <- lane4 byte 0, byte 1 <- w byte J, bytes 2..3 <- 0x00
  constexpr uint32_t sel = 0x0C0C0400u + (static_cast<uint32_t>(J) << 8);
  return lds0_u32(__builtin_amdgcn_perm(w, lane4, sel));
}

// bf16 bits (round to nearest even) of a finite binary32 pattern, usable at compile time.
constexpr uint32_t bf16_bits_rne(uint32_t b) { return (b + 0x7FFFu + ((b >> 16) & 1u)) >> 16; }

// Fill the table from a workgroup of exactly 16 wavefronts; the caller's next barrier
// publishes it.  Wavefront v writes the bytes whose low code is v: byte = v + 16*j has
// high code j, a compile-time constant, so an entry costs one OR and one LDS store.
__device__ __forceinline__ void fill_pair_table(uint32_t *table, int wave, int lane) {
  const uint32_t lo = bf16_bits_rne(kLutBits[wave]);
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const uint32_t hi = bf16_bits_rne(kLevelBits[j]) << 16;
    table[((wave + 16 * j) << 6) + lane] = lo | hi;
  }
}

__device__ __forceinline__ uint4 lds0_u128(uint32_t addr) {
  const U32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) U32x4 *>(addr);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// Compute units of the current device (256 on an MI355X), cached after the first call.
inline int device_cu_count() {
  static int cached = [] {
    constexpr int kDefault = 256;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
      (void)hipGetLastError();
      return kDefault;
    }
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n < 1) {
      (void)hipGetLastError();
      return kDefault;
    }
    return n;
  }();
  return cached;
}

inline int launch_rc() { return hipGetLastError() == hipSuccess ? 0 : -6; }

}  // namespace chr

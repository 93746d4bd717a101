/* CPU oracle for the group-64 NF4 codec and the packed linear layer.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library or its Python
 * wrappers may link, load or call this file; it exists so that tests (and the
 * bench's cpu_baseline leg) have an independent CPU answer to compare the HIP
 * kernels with.
 *
 * Each function restates, in plain C, the reference routine it cites
 * (paths relative to the reference checkout):
 *
 *   or_f16_to_f32      internal/f16/f16.go:59-85   (ToFloat32)
 *   or_f32_to_f16      internal/f16/f16.go:8-57    (FromFloat32, RNE)
 *   or_bf16_to_f32     internal/f16/f16.go:88-91   (FromBF16Bits)
 *   or_f32_to_bf16     internal/f16/f16.go:93-106  (ToBF16Bits, RNE)
 *   or_nf4_lut         internal/nf4/nf4.go:18-35   (NF4 table)
 *   or_nf4_encode      internal/nf4/nf4.go:46-82, 129-185
 *   or_nf4_decode      internal/nf4/nf4.go:85-121
 *   or_matmul_f32      gpu/tests/nf4_oracle.py:134-138 (float32 W_hat @ x)
 *   or_linear_two_pass gpu/decodev2/linear.py:128-133  (decode, then matmul)
 *
 * Pinned by: the golden vectors of internal/nf4/nf4_test.go and
 * internal/f16/f16_test.go (tests/test_oracle_golden.py), all 65,536 binary16
 * patterns against numpy.float16, a bf16 grid against torch, the 15 midpoints
 * of docs/spec/nf4.md section 2.3, and an independent numpy restatement.
 *
 * Build: see oracle/Makefile.  -ffp-contract=off keeps every float operation
 * a separately rounded binary32 operation, as the Go code is on amd64.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define OR_GROUP 64

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  return u;
}

static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

/* The sixteen levels, written as their binary32 bit patterns
 * (internal/nf4/nf4_test.go:12-29 lists the same words). */
static const uint32_t kLutBits[16] = {
    0xBF800000u, 0xBF3239B1u, 0xBF066B30u, 0xBECA32A0u, 0xBE91A24Du, 0xBE3D353Fu,
    0xBDBA7871u, 0x00000000u, 0x3DA2FAFFu, 0x3E24CAE3u, 0x3E7C04DDu, 0x3EAD033Au,
    0x3EE1A4B8u, 0x3F1007ABu, 0x3F3913B3u, 0x3F800000u,
};

void or_nf4_lut(float out[16]) {
  for (int i = 0; i < 16; ++i) {
    out[i] = bits_f32(kLutBits[i]);
  }
}

/* binary16 -> binary32, exact (subnormals normalised, Inf/NaN payload kept). */
float or_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t out;
  if (exp == 0) {
    if (man == 0) {
      out = sign;
    } else {
      uint32_t e = 127 - 15 + 1;
      while ((man & 0x400u) == 0) {
        man <<= 1;
        --e;
      }
      out = sign | (e << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 0x1Fu) {
    out = sign | 0x7F800000u | (man << 13);
  } else {
    out = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  return bits_f32(out);
}

/* binary32 -> binary16, round to nearest even; overflow -> Inf, tiny -> 0 or
 * a subnormal; NaN keeps a non-zero mantissa. */
uint16_t or_f32_to_f16(float f) {
  const uint32_t b = f32_bits(f);
  const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
  const int exp = (int)((b >> 23) & 0xFFu);
  uint32_t man = b & 0x7FFFFFu;
  if (exp == 0xFF) {
    if (man != 0) {
      uint16_t n = (uint16_t)(man >> 13);
      if (n == 0) {
        n = 1;
      }
      return (uint16_t)(sign | 0x7C00u | n);
    }
    return (uint16_t)(sign | 0x7C00u);
  }
  const int e = exp - 127 + 15;
  if (e >= 0x1F) {
    return (uint16_t)(sign | 0x7C00u);
  }
  if (e <= 0) {
    if (e < -10) {
      return sign;
    }
    man |= 1u << 23;
    const uint32_t shift = (uint32_t)(14 - e);
    const uint32_t round = (man >> (shift - 1)) & 1u;
    const uint32_t tail = man & ((1u << (shift - 1)) - 1u);
    uint32_t m = man >> shift;
    if (round != 0 && (tail != 0 || (m & 1u) != 0)) {
      ++m;
    }
    return (uint16_t)(sign | (uint16_t)m);
  }
  uint16_t half = (uint16_t)(sign | (uint16_t)(e << 10) | (uint16_t)(man >> 13));
  const uint32_t rem = man & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u) != 0)) {
    ++half; /* a carry out of the mantissa bumps the exponent, up to Inf */
  }
  return half;
}

float or_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t or_f32_to_bf16(float f) {
  uint32_t b = f32_bits(f);
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) {
    uint16_t n = (uint16_t)(b >> 16);
    if ((n & 0x7Fu) == 0) {
      n |= 1;
    }
    return n;
  }
  const uint32_t lsb = (b >> 16) & 1u;
  b += 0x7FFFu + lsb;
  return (uint16_t)(b >> 16);
}

static int k_padded(int k) { return ((k + OR_GROUP - 1) / OR_GROUP) * OR_GROUP; }

static int is_finite32(float x) {
  return (f32_bits(x) & 0x7F800000u) != 0x7F800000u;
}

/* Nearest level by squared distance in binary32, first minimum wins
 * (internal/nf4/nf4.go:168-181). */
static uint8_t nearest_level(float u, const float *lut) {
  uint8_t best_j = 0;
  float d = u - lut[0];
  float best = d * d;
  for (int j = 1; j < 16; ++j) {
    d = u - lut[j];
    const float d2 = d * d;
    if (d2 < best) {
      best = d2;
      best_j = (uint8_t)j;
    }
  }
  return best_j;
}

/* One group of 64.  Returns 0, or -2 for a non-finite weight, -3 for a scale
 * that is still not finite-positive after the clamp. */
static int encode_group(const float *g, const float *lut, uint8_t *idx,
                        uint16_t *s16_out) {
  float s32 = 0.0f;
  for (int i = 0; i < OR_GROUP; ++i) {
    if (!is_finite32(g[i])) {
      return -2;
    }
    const float a = fabsf(g[i]);
    if (a > s32) {
      s32 = a;
    }
  }
  if (s32 == 0.0f) {
    s32 = 1.0f;
  }
  uint16_t s16 = or_f32_to_f16(s32);
  float s = or_f16_to_f32(s16);
  if (!is_finite32(s) || !(s > 0.0f)) {
    /* binary16 flushed a tiny scale to zero or overflowed a huge one:
     * the tiny group becomes a zero group (scale 1), the huge one clamps
     * to the largest finite binary16 (internal/nf4/nf4.go:145-156). */
    s32 = (s32 > 65504.0f) ? 65504.0f : 1.0f;
    s16 = or_f32_to_f16(s32);
    s = or_f16_to_f32(s16);
  }
  if (!is_finite32(s) || !(s > 0.0f)) {
    return -3;
  }
  for (int i = 0; i < OR_GROUP; ++i) {
    float u = g[i] / s;
    if (u > 1.0f) {
      u = 1.0f;
    } else if (u < -1.0f) {
      u = -1.0f;
    }
    idx[i] = nearest_level(u, lut);
  }
  *s16_out = s16;
  return 0;
}

/* W[n_out, n_in] row-major float32 -> data[n_out, K_pad/2], scale[n_out, K_pad/64].
 * Low nibble = even column.  Columns past n_in are treated as zero weights.
 * Returns 0; -1 empty shape; -2 non-finite weight; -3 bad scale. */
int or_nf4_encode(const float *w, int n_out, int n_in, uint8_t *data,
                  uint16_t *scale) {
  if (n_out < 1 || n_in < 1) {
    return -1;
  }
  float lut[16];
  or_nf4_lut(lut);
  const int kp = k_padded(n_in);
  const int ng = kp / OR_GROUP;
  int rc_all = 0;
#pragma omp parallel for schedule(static) reduction(min : rc_all)
  for (int r = 0; r < n_out; ++r) {
    float grp[OR_GROUP];
    uint8_t idx[OR_GROUP];
    const float *row = w + (size_t)r * (size_t)n_in;
    for (int g = 0; g < ng; ++g) {
      for (int k = 0; k < OR_GROUP; ++k) {
        const int c = g * OR_GROUP + k;
        grp[k] = (c < n_in) ? row[c] : 0.0f;
      }
      uint16_t s16 = 0;
      const int rc = encode_group(grp, lut, idx, &s16);
      if (rc != 0) {
        if (rc < rc_all) {
          rc_all = rc;
        }
        continue;
      }
      scale[(size_t)r * ng + g] = s16;
      uint8_t *dst = data + (size_t)r * (kp / 2) + (size_t)g * (OR_GROUP / 2);
      for (int k = 0; k < OR_GROUP / 2; ++k) {
        dst[k] = (uint8_t)((idx[2 * k + 1] << 4) | idx[2 * k]);
      }
    }
  }
  return rc_all;
}

/* data/scale -> W_hat[n_out, n_in] float32, one binary32 multiply per weight,
 * padding columns dropped.  Returns 0 or -1 for an empty shape. */
int or_nf4_decode(const uint8_t *data, const uint16_t *scale, int n_out, int n_in,
                  float *out) {
  if (n_out < 1 || n_in < 1) {
    return -1;
  }
  float lut[16];
  or_nf4_lut(lut);
  const int kp = k_padded(n_in);
  const int ng = kp / OR_GROUP;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < n_out; ++r) {
    for (int g = 0; g < ng; ++g) {
      const float s = or_f16_to_f32(scale[(size_t)r * ng + g]);
      const uint8_t *src = data + (size_t)r * (kp / 2) + (size_t)g * (OR_GROUP / 2);
      for (int k = 0; k < OR_GROUP; ++k) {
        const int c = g * OR_GROUP + k;
        if (c >= n_in) {
          continue;
        }
        const uint8_t b = src[k / 2];
        const uint8_t nib = (k % 2 == 0) ? (uint8_t)(b & 0x0F) : (uint8_t)(b >> 4);
        out[(size_t)r * n_in + c] = lut[nib] * s;
      }
    }
  }
  return 0;
}

/* y[M,N] = w[M,K] @ x[K,N], all float32 row-major, float32 accumulation in
 * index order of k.  The reference's CPU matmul is numpy's (BLAS order); any
 * float32 order is inside the tolerance the GEMV/GEMM tests state. */
void or_matmul_f32(const float *w, const float *x, int m, int k, int n, float *y) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < m; ++r) {
    const float *wr = w + (size_t)r * k;
    float *yr = y + (size_t)r * n;
    for (int j = 0; j < n; ++j) {
      yr[j] = 0.0f;
    }
    for (int c = 0; c < k; ++c) {
      const float wv = wr[c];
      const float *xr = x + (size_t)c * n;
      for (int j = 0; j < n; ++j) {
        yr[j] += wv * xr[j];
      }
    }
  }
}

/* Same product accumulated in binary64: used to report the float32 oracle's
 * own rounding noise next to the kernel error. */
void or_matmul_f64(const float *w, const float *x, int m, int k, int n, double *y) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < m; ++r) {
    const float *wr = w + (size_t)r * k;
    double *yr = y + (size_t)r * n;
    for (int j = 0; j < n; ++j) {
      yr[j] = 0.0;
    }
    for (int c = 0; c < k; ++c) {
      const double wv = (double)wr[c];
      const float *xr = x + (size_t)c * n;
      for (int j = 0; j < n; ++j) {
        yr[j] += wv * (double)xr[j];
      }
    }
  }
}

/* The reference's CPU linear: decode the whole matrix to float32 (pass 1),
 * then a float32 matmul (pass 2).  scratch holds m*k floats. */
int or_linear_two_pass(const uint8_t *data, const uint16_t *scale, int m, int k,
                       const float *x, int n, float *scratch, float *y) {
  const int rc = or_nf4_decode(data, scale, m, k, scratch);
  if (rc != 0) {
    return rc;
  }
  or_matmul_f32(scratch, x, m, k, n, y);
  return 0;
}

/* Fused decode+dot for N=1, reported beside the two-pass baseline. */
void or_gemv_fused(const uint8_t *data, const uint16_t *scale, int m, int k,
                   const float *x, float *y) {
  float lut[16];
  or_nf4_lut(lut);
  const int kp = k_padded(k);
  const int ng = kp / OR_GROUP;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < m; ++r) {
    float acc = 0.0f;
    for (int g = 0; g < ng; ++g) {
      const float s = or_f16_to_f32(scale[(size_t)r * ng + g]);
      const uint8_t *src = data + (size_t)r * (kp / 2) + (size_t)g * (OR_GROUP / 2);
      const int lim = (k - g * OR_GROUP < OR_GROUP) ? (k - g * OR_GROUP) : OR_GROUP;
      for (int c = 0; c < lim; ++c) {
        const uint8_t b = src[c / 2];
        const uint8_t nib = (c % 2 == 0) ? (uint8_t)(b & 0x0F) : (uint8_t)(b >> 4);
        acc += (lut[nib] * s) * x[g * OR_GROUP + c];
      }
    }
    y[r] = acc;
  }
}

void or_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) {
    omp_set_num_threads(n);
  }
#else
  (void)n;
#endif
}

int or_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

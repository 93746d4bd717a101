// A caller of the NF4 library written the way the reference's own host code calls its
// kernels: plain C types, hipMalloc'd buffers, no Python and no torch anywhere in the
// process.  It quantises a random matrix on the device, then checks the decode, the N=1
// GEMV and the 8-column GEMM against arithmetic done right here on the host from the
// packed bytes the library produced.
//
//   host_check --host-only   argument checks and the launch plan; touches no GPU
//   host_check               everything, on device 0
//
// Exit status 0 and a last line "host_check: OK" mean every check passed.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "chr_nf4_amd.h"

namespace {

int failures = 0;

#define EXPECT(cond, ...)                          \
  do {                                             \
    if (!(cond)) {                                 \
      ++failures;                                  \
      std::printf("FAIL %s:%d  ", __FILE__, __LINE__); \
      std::printf(__VA_ARGS__);                    \
      std::printf("\n");                           \
    }                                              \
  } while (0)

#define HIP_OK(call)                                                              \
  do {                                                                            \
    hipError_t e_ = (call);                                                       \
    if (e_ != hipSuccess) {                                                       \
      std::printf("host_check: %s -> %s\n", #call, hipGetErrorString(e_));        \
      std::exit(2);                                                               \
    }                                                                             \
  } while (0)

// The sixteen NF4 levels as binary32 bit patterns (the published QLoRA table).
const uint32_t kLevelBits[16] = {
    0xBF800000u, 0xBF3239B1u, 0xBF066B30u, 0xBECA32A0u, 0xBE91A24Du, 0xBE3D353Fu,
    0xBDBA7871u, 0x00000000u, 0x3DA2FAFFu, 0x3E24CAE3u, 0x3E7C04DDu, 0x3EAD033Au,
    0x3EE1A4B8u, 0x3F1007ABu, 0x3F3913B3u, 0x3F800000u};

float from_bits(uint32_t b) {
  float f;
  std::memcpy(&f, &b, 4);
  return f;
}
uint32_t to_bits(float f) {
  uint32_t b;
  std::memcpy(&b, &f, 4);
  return b;
}

float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const int exp = (h >> 10) & 0x1F;
  const uint32_t man = h & 0x3FFu;
  if (exp == 0) return from_bits(sign) + (sign ? -1.0f : 1.0f) * std::ldexp((float)man, -24);
  if (exp == 31) return from_bits(sign | 0x7F800000u | (man << 13));
  return from_bits(sign | ((uint32_t)(exp + 112) << 23) | (man << 13));
}

uint16_t float_to_bf16(float f) {
  uint32_t b = to_bits(f);
  b += 0x7FFFu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}
float bf16_to_float(uint16_t h) { return from_bits((uint32_t)h << 16); }

// xorshift: the same inputs on every run.
struct Rng {
  uint64_t s;
  float uniform() {  // in (-1, 1)
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return (float)((double)(s >> 11) / 9007199254740992.0 * 2.0 - 1.0);
  }
};

void host_only() {
  chr_nf4_dev_t w{5120, 5120, 5120, nullptr, nullptr};
  chr_nf4_plan_t p{};
  EXPECT(chr_nf4_gemm_plan(&w, 1, 1, &p) == 0, "plan N=1");
  EXPECT(p.path == 1 && p.grid_y == 1 && p.ws_floats == 0, "N=1 plans the GEMV tile (path %d)", p.path);
  EXPECT(chr_nf4_gemm_plan(&w, 32, 1, &p) == 0, "plan N=32");
  EXPECT(p.path == 3 && p.ctas == p.grid_x * p.grid_y, "N=32 plans the 32-column MFMA tile");
  EXPECT(p.grid_y == 1 ? p.ws_floats == 0 : p.ws_floats >= (int64_t)p.grid_y * 5120 * 32,
         "workspace covers the split-K partials");
  EXPECT(chr_nf4_gemm_plan(&w, 0, 1, &p) == -2, "N=0 is out of range");
  EXPECT(chr_nf4_gemm_plan(&w, 65, 1, &p) == -2, "N=65 is out of range");
  EXPECT(chr_nf4_gemm_plan(nullptr, 1, 1, &p) == -1, "null descriptor");
  chr_nf4_dev_t bad{64, 100, 64, nullptr, nullptr};
  EXPECT(chr_nf4_gemm_plan(&bad, 1, 1, &p) == -4, "K_pad below K");
  EXPECT(chr_nf4_gemv(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0.f) == -1, "null gemv");
  EXPECT(chr_nf4_gemm(&w, nullptr, nullptr, 4, nullptr) == -1, "null operands");
}

void on_device() {
  const int M = 192, K = 1000, K_pad = 1024, N = 8;
  const int groups = K_pad / 64;
  Rng rng{0x9E3779B97F4A7C15ull};

  std::vector<float> W((size_t)M * K);
  for (auto &v : W) v = rng.uniform() * 0.05f;
  std::vector<uint16_t> x1(K), xn((size_t)K * N);
  for (auto &v : x1) v = float_to_bf16(rng.uniform());
  for (auto &v : xn) v = float_to_bf16(rng.uniform());

  HIP_OK(hipSetDevice(0));
  float *dW, *dOut, *dWs;
  uint8_t *dPacked;
  uint16_t *dScale, *dX1, *dXn, *dY1, *dYn;
  int32_t *dStatus;
  HIP_OK(hipMalloc(&dW, W.size() * 4));
  HIP_OK(hipMalloc(&dOut, W.size() * 4));
  HIP_OK(hipMalloc(&dPacked, (size_t)M * K_pad / 2));
  HIP_OK(hipMalloc(&dScale, (size_t)M * groups * 2));
  HIP_OK(hipMalloc(&dX1, K * 2));
  HIP_OK(hipMalloc(&dXn, (size_t)K * N * 2));
  HIP_OK(hipMalloc(&dY1, M * 2));
  HIP_OK(hipMalloc(&dYn, (size_t)M * N * 2));
  HIP_OK(hipMalloc(&dStatus, 4));
  HIP_OK(hipMemset(dStatus, 0, 4));
  HIP_OK(hipMemcpy(dW, W.data(), W.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dX1, x1.data(), K * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dXn, xn.data(), (size_t)K * N * 2, hipMemcpyHostToDevice));

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  chr_nf4_dev_t w{M, K, K_pad, dPacked, dScale};

  // Encode on the device, then bring the packed form back.
  EXPECT(chr_nf4_quantize(dW, &w, dStatus, stream) == 0, "quantize");
  EXPECT(chr_nf4_dequant(&w, dOut, stream) == 0, "dequant");
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<uint8_t> packed((size_t)M * K_pad / 2);
  std::vector<uint16_t> scale((size_t)M * groups);
  std::vector<float> out(W.size());
  int32_t status = -1;
  HIP_OK(hipMemcpy(packed.data(), dPacked, packed.size(), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(scale.data(), dScale, scale.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(out.data(), dOut, out.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&status, dStatus, 4, hipMemcpyDeviceToHost));
  EXPECT(status == 0, "every weight was finite, status %d", status);

  // Host decode of those bytes: low nibble = even column, one fp32 multiply.
  std::vector<float> deq((size_t)M * K);
  size_t mismatched = 0;
  double worst_quant = 0.0;
  for (int r = 0; r < M; ++r)
    for (int c = 0; c < K; ++c) {
      const uint8_t b = packed[(size_t)r * (K_pad / 2) + c / 2];
      const int code = (c & 1) ? (b >> 4) : (b & 0x0F);
      const float s = half_to_float(scale[(size_t)r * groups + c / 64]);
      const float v = from_bits(kLevelBits[code]) * s;
      deq[(size_t)r * K + c] = v;
      mismatched += to_bits(v) != to_bits(out[(size_t)r * K + c]);
      // A 4-bit code cannot be further from the weight than half the widest level gap.
      const double err = std::fabs((double)v - W[(size_t)r * K + c]);
      if (s > 0.f && err / s > worst_quant) worst_quant = err / s;
    }
  EXPECT(mismatched == 0, "device decode differs from the host decode in %zu weights", mismatched);
  EXPECT(worst_quant <= 0.16, "quantisation error %.3f of the group scale", worst_quant);
  // Columns K..K_pad are padding and must hold the code of 0.0 (7).
  size_t bad_pad = 0;
  for (int r = 0; r < M; ++r)
    for (int c = K; c < K_pad; ++c) {
      const uint8_t b = packed[(size_t)r * (K_pad / 2) + c / 2];
      bad_pad += ((c & 1) ? (b >> 4) : (b & 0x0F)) != 7;
    }
  EXPECT(bad_pad == 0, "%zu padding codes are not the zero level", bad_pad);

  // N=1 GEMV and the 8-column GEMM (with and without a split-K workspace).
  chr_nf4_plan_t plan{};
  EXPECT(chr_nf4_gemm_plan(&w, N, 1, &plan) == 0, "plan");
  const int64_t ws_floats = plan.ws_floats > 0 ? plan.ws_floats : 1;
  HIP_OK(hipMalloc(&dWs, ws_floats * 4));

  std::vector<uint16_t> y1(M), yn((size_t)M * N), yw((size_t)M * N);
  EXPECT(chr_nf4_gemv(&w, dX1, dY1, stream, nullptr, nullptr, 0.f) == 0, "gemv");
  EXPECT(chr_nf4_gemm(&w, dXn, dYn, N, stream) == 0, "gemm");
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(y1.data(), dY1, M * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(yn.data(), dYn, yn.size() * 2, hipMemcpyDeviceToHost));
  EXPECT(chr_nf4_gemm_ws(&w, dXn, dYn, N, dWs, ws_floats, stream) == 0, "gemm_ws");
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(yw.data(), dYn, yw.size() * 2, hipMemcpyDeviceToHost));

  auto max_rel = [&](const std::vector<uint16_t> &y, const std::vector<uint16_t> &x, int n) {
    double worst = 0.0, peak = 0.0;
    std::vector<double> ref((size_t)M * n);
    for (int r = 0; r < M; ++r)
      for (int j = 0; j < n; ++j) {
        double acc = 0.0;
        for (int c = 0; c < K; ++c)
          acc += (double)deq[(size_t)r * K + c] * bf16_to_float(x[(size_t)c * n + j]);
        ref[(size_t)r * n + j] = acc;
        peak = std::fmax(peak, std::fabs(acc));
      }
    for (size_t i = 0; i < ref.size(); ++i)
      worst = std::fmax(worst, std::fabs(bf16_to_float(y[i]) - ref[i]) / peak);
    return worst;
  };
  const double e1 = max_rel(y1, x1, 1), en = max_rel(yn, xn, N), ew = max_rel(yw, xn, N);
  std::printf("gemv max-rel %.2e, gemm %.2e, gemm_ws %.2e (split_k %d)\n", e1, en, ew, plan.grid_y);
  EXPECT(e1 <= 1e-2, "gemv max-rel %.3e", e1);
  EXPECT(en <= 1e-2, "gemm max-rel %.3e", en);
  EXPECT(ew <= 1e-2, "gemm_ws max-rel %.3e", ew);

  // The sum of squares handed from the launch that writes a vector to the launch that
  // normalises it: the GEMV leaves the parts for its y (same y, bit for bit), a GEMV with a
  // norm takes mean(x^2) from parts, and a launch that can serve neither says -8.
  {
    const int n_parts = chr_dv2_sumsq_parts();
    EXPECT(n_parts >= 64 && n_parts % 4 == 0, "parts %d", n_parts);
    float *dParts;
    uint16_t *dG, *dY2;
    HIP_OK(hipMalloc(&dParts, n_parts * 4));
    HIP_OK(hipMalloc(&dG, K * 2));
    HIP_OK(hipMalloc(&dY2, M * 2));
    EXPECT(chr_dv2_sumsq_ok(M, K, K_pad, 0) == 1, "a ragged K runs on a kernel that stages x");
    EXPECT(chr_dv2_gemv_sumsq(&w, dX1, dY2, stream, nullptr, nullptr, 0.f, nullptr, dParts) == 0,
           "gemv with sumsq_out");
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> parts(n_parts);
    std::vector<uint16_t> y2(M);
    HIP_OK(hipMemcpy(parts.data(), dParts, n_parts * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(y2.data(), dY2, M * 2, hipMemcpyDeviceToHost));
    EXPECT(y2 == y1, "sumsq_out changed y");
    double left = 0.0, want = 0.0;
    for (float v : parts) left += v;
    for (uint16_t v : y2) want += (double)bf16_to_float(v) * bf16_to_float(v);
    EXPECT(std::fabs(left - want) <= 1e-5 * want, "parts add up to %.6g, y^2 to %.6g", left, want);

    std::vector<uint16_t> g(K, float_to_bf16(1.0f));
    double xx = 0.0;
    for (uint16_t v : x1) xx += (double)bf16_to_float(v) * bf16_to_float(v);
    std::fill(parts.begin(), parts.end(), 0.f);
    parts[0] = (float)xx;
    HIP_OK(hipMemcpy(dG, g.data(), K * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dParts, parts.data(), n_parts * 4, hipMemcpyHostToDevice));
    EXPECT(chr_nf4_gemv(&w, dX1, dY1, stream, nullptr, dG, 1e-6f) == 0, "gemv with a norm");
    EXPECT(chr_dv2_gemv_sumsq(&w, dX1, dY2, stream, nullptr, dG, 1e-6f, dParts, nullptr) == 0,
           "gemv with a norm and sumsq_in");
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> ya(M), yb(M);
    HIP_OK(hipMemcpy(ya.data(), dY1, M * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(yb.data(), dY2, M * 2, hipMemcpyDeviceToHost));
    double peak = 0.0, apart = 0.0;
    for (int r = 0; r < M; ++r) {
      peak = std::fmax(peak, std::fabs(bf16_to_float(ya[r])));
      apart = std::fmax(apart, std::fabs(bf16_to_float(ya[r]) - bf16_to_float(yb[r])));
    }
    EXPECT(peak > 0.0 && apart <= peak / 128, "handed sum: %.3g apart at a peak of %.3g", apart, peak);
    EXPECT(chr_dv2_gemv_sumsq(&w, dX1, dY2, stream, nullptr, nullptr, 0.f, dParts, nullptr) == -8,
           "sumsq_in without a norm");
    HIP_OK(hipStreamSynchronize(stream));
    for (void *p : {(void *)dParts, (void *)dG, (void *)dY2}) HIP_OK(hipFree(p));
  }

  // Refusals that must come back as codes, not as faults.
  EXPECT(chr_nf4_gemm(&w, dXn, dYn, 33, stream) == -2, "N=33 has no tile");
  if (plan.ws_floats > 1)
    EXPECT(chr_nf4_gemm_ws(&w, dXn, dYn, N, dWs, plan.ws_floats - 1, stream) == -7,
           "a workspace one float short of the plan is refused");
  HIP_OK(hipStreamSynchronize(stream));

  HIP_OK(hipStreamDestroy(stream));
  for (void *p : {(void *)dW, (void *)dOut, (void *)dPacked, (void *)dScale, (void *)dX1,
                  (void *)dXn, (void *)dY1, (void *)dYn, (void *)dStatus, (void *)dWs})
    HIP_OK(hipFree(p));
}

}  // namespace

int main(int argc, char **argv) {
  const bool host = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
  host_only();
  if (!host) on_device();
  if (failures) {
    std::printf("host_check: %d check(s) failed\n", failures);
    return 1;
  }
  std::printf("host_check: OK\n");
  return 0;
}

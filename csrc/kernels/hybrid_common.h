// Helpers shared by the kernel files of the hybrid decoder designs (hybrid.hip, hybrid_moe.hip).
#pragma once
#include "common.h"

namespace {

// An activation-typed buffer (fp32 or bf16, a launch-time flag) read and written as floats.
template <bool F32>
struct Act;
template <>
struct Act<true> {
  typedef float type;
  static LC_DEVICE float load(const float* p, size_t i) { return p[i]; }
  static LC_DEVICE void store(float* p, size_t i, float v) { p[i] = v; }
};
template <>
struct Act<false> {
  typedef bf16_t type;
  static LC_DEVICE float load(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
  static LC_DEVICE void store(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }
};

LC_DEVICE float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
LC_DEVICE float siluf_(float x) { return x / (1.f + expf(-x)); }
// log sigmoid(z) = min(z, 0) - log1p(exp(-|z|))
LC_DEVICE float logsigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

}  // namespace

// Element access of the fp32-residual kernel set: activations are bf16 (raw bits) or fp32, arithmetic is fp32.
#pragma once
#include "../common.h"

namespace lwc {

template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  static LWC_DEVICE float ld(const bf16_t* p) { return bf2f(*p); }
  static LWC_DEVICE void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <> struct Elem<float> {
  static LWC_DEVICE float ld(const float* p) { return *p; }
  static LWC_DEVICE void st(float* p, float v) { *p = v; }
};

LWC_DEVICE float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
LWC_DEVICE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
LWC_DEVICE float silu_f(float x) { return x / (1.0f + expf(-x)); }
LWC_DEVICE float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

}  // namespace lwc

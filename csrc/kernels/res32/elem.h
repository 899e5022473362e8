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

// four consecutive elements (16 bytes of fp32, 8 bytes of bf16) <-> four floats
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static LWC_DEVICE float4v ld(const float* p) { return *reinterpret_cast<const float4v*>(p); }
  static LWC_DEVICE void st(float* p, float4v v) { *reinterpret_cast<float4v*>(p) = v; }
};
template <> struct Vec4<bf16_t> {
  static LWC_DEVICE float4v ld(const bf16_t* p) {
    const uint2v w = *reinterpret_cast<const uint2v*>(p);
    return float4v{__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xffff0000u), __uint_as_float(w[1] << 16),
                   __uint_as_float(w[1] & 0xffff0000u)};
  }
  static LWC_DEVICE void st(bf16_t* p, float4v v) {
    *reinterpret_cast<uint2v*>(p) = uint2v{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  }
};
inline bool aligned_to(const void* p, int bytes) { return ((uintptr_t)p & (uintptr_t)(bytes - 1)) == 0; }

LWC_DEVICE float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
LWC_DEVICE float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
LWC_DEVICE float silu_f(float x) { return x / (1.0f + expf(-x)); }
LWC_DEVICE float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

}  // namespace lwc

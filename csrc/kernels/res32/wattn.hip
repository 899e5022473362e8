// Sliding-window attention with a logarithmic distance bias over a paged K/V cache (gfx950, wave64).
//
//   score(i, j) = q_i . k_j - r1_h * ln(1 + r2_h * (i - j))        for 0 <= i - j < window
//   out_i       = softmax_j(score) . v_j
// q arrives in fp32 already multiplied by the head's softmax scale; K rows have D elements, V rows Dv (any sizes,
// D != Dv allowed), G key/value heads serve H query heads (head h reads group h / (H / G)).  Scores, the softmax
// and the weighted sum are fp32 whatever the cache's element type (bf16 or fp32).
//
// Cache layout (one layer): K [num_blocks, block_size, G * D], V [num_blocks, block_size, G * Dv], with a
// block stride given separately (the layers of a model share one pool).
//
// Rows are query tokens.  Row t belongs to table row `item`: t itself when cu_q is null (decode: one token
// per sequence), else the item with cu_q[item] <= t < cu_q[item + 1] (a portion of a prompt); its position in
// the sequence is positions[t], and every key it may see is already in the cache.
//
// window_attn_kernel: one wave per (row, head); lanes over 64 keys for the scores, an online softmax per
// 64-key step, then lanes over the value dimension (several keys side by side when Dv < 64).
#include "../common.h"

namespace lwc {
namespace {

template <typename CT> struct KLoad;
template <> struct KLoad<bf16_t> {
  static constexpr int kVec = 8;
  static LWC_DEVICE float dot(const bf16_t* k, const float* q, int D) {
    float acc = 0.f;
    if ((D & 7) == 0 && ((uintptr_t)k & 15) == 0) {
      for (int d = 0; d < D; d += 8) {
        const uint4v kv = *reinterpret_cast<const uint4v*>(k + d);
        float f[8];
        unpack8(kv, f);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += q[d + e] * f[e];
      }
    } else {
      for (int d = 0; d < D; ++d) acc += q[d] * bf2f(k[d]);
    }
    return acc;
  }
  static LWC_DEVICE float ld(const bf16_t* p) { return bf2f(*p); }
  static LWC_DEVICE void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <> struct KLoad<float> {
  static LWC_DEVICE float dot(const float* k, const float* q, int D) {
    float acc = 0.f;
    if ((D & 3) == 0 && ((uintptr_t)k & 15) == 0) {
      for (int d = 0; d < D; d += 4) {
        const float4v kv = *reinterpret_cast<const float4v*>(k + d);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc += q[d + e] * kv[e];
      }
    } else {
      for (int d = 0; d < D; ++d) acc += q[d] * k[d];
    }
    return acc;
  }
  static LWC_DEVICE float ld(const float* p) { return *p; }
  static LWC_DEVICE void st(float* p, float v) { *p = v; }
};

constexpr int kMaxSlots = 4;  // value dimension <= 256

template <typename CT>
__global__ void __launch_bounds__(64)
window_attn_kernel(const float* __restrict__ q, const CT* __restrict__ k_cache, const CT* __restrict__ v_cache,
                   long long kb_stride, long long vb_stride, int block_size, const int* __restrict__ positions,
                   const int* __restrict__ cu_q, int n_items, const int* __restrict__ block_tables, int bt_width,
                   const float* __restrict__ r1, const float* __restrict__ r2, int window, CT* __restrict__ out,
                   int ldo, int H, int G, int D, int Dv) {
  extern __shared__ float q_s[];  // [D]
  __shared__ float p_s[64];
  __shared__ long long vo_s[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  int item = t;
  if (cu_q) {
    int lo = 0, hi = n_items - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    item = lo;
  }
  const int* table = block_tables + (size_t)item * bt_width;
  const int i = positions[t];
  const int g = h / (H / G);
  for (int d = lane; d < D; d += 64) q_s[d] = q[((size_t)t * H + h) * D + d];
  __syncthreads();
  const float r1h = r1[h], r2h = r2[h];
  int DvP = 64;
  if (Dv < 64) {
    DvP = 1;
    while (DvP < Dv) DvP <<= 1;
  }
  const int kpar = 64 / DvP, dvl = lane % DvP, kp = lane / DvP;
  float o[kMaxSlots] = {0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int j_lo = max(0, i - window + 1);
  for (int j0 = j_lo; j0 <= i; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= i;
    float s = -INFINITY;
    long long vo = 0;
    if (valid) {
      const long long blk = table[j / block_size];
      const long long off = j % block_size;
      const CT* kr = k_cache + blk * kb_stride + (off * G + g) * D;
      s = KLoad<CT>::dot(kr, q_s, D) - r1h * log1pf(r2h * (float)(i - j));
      vo = blk * vb_stride + (off * G + g) * Dv;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    vo_s[lane] = vo;
    __syncthreads();
    const int nkeys = min(64, i - j0 + 1);
#pragma unroll
    for (int ns = 0; ns < kMaxSlots; ++ns) o[ns] *= alpha;
    for (int jj = kp; jj < nkeys; jj += kpar) {
      const float pj = p_s[jj];
      const CT* vr = v_cache + vo_s[jj];
#pragma unroll
      for (int ns = 0; ns < kMaxSlots; ++ns) {
        const int dv = ns * 64 + dvl;
        if (dv < Dv) o[ns] += pj * KLoad<CT>::ld(vr + dv);
      }
    }
  }
  for (int off = DvP; off < 64; off <<= 1) o[0] += __shfl_xor(o[0], off, 64);
  if (kp == 0) {
    const float inv = 1.0f / l;
    CT* orow = out + (size_t)t * ldo + (size_t)h * Dv;
#pragma unroll
    for (int ns = 0; ns < kMaxSlots; ++ns) {
      const int dv = ns * 64 + dvl;
      if (dv < Dv) KLoad<CT>::st(orow + dv, o[ns] * inv);
    }
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_window_attn(const float* q, const void* k_cache, const void* v_cache, long long kb_stride,
                               long long vb_stride, int block_size, const int* positions, const int* cu_q, int n_items,
                               const int* block_tables, int bt_width, const float* r1, const float* r2, int window,
                               void* out, int ldo, int T, int H, int G, int D, int Dv, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (Dv > 64 * kMaxSlots || D > 8192 || H % G != 0) return -1;
  const dim3 grid(T, H);
  const size_t shm = (size_t)D * sizeof(float);
  if (f32)
    window_attn_kernel<float><<<grid, 64, shm, s>>>(q, (const float*)k_cache, (const float*)v_cache, kb_stride, vb_stride,
                                                    block_size, positions, cu_q, n_items, block_tables, bt_width, r1, r2,
                                                    window, (float*)out, ldo, H, G, D, Dv);
  else
    window_attn_kernel<bf16_t><<<grid, 64, shm, s>>>(q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, kb_stride,
                                                     vb_stride, block_size, positions, cu_q, n_items, block_tables,
                                                     bt_width, r1, r2, window, (bf16_t*)out, ldo, H, G, D, Dv);
  return (int)hipGetLastError();
}

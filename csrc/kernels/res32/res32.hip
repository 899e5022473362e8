// Kernels for decoder designs that carry their residual stream in fp32 (gfx950, wave64).
//
// The activations between the kernels (AT) are bf16 or fp32 (one template argument); the residual stream,
// every statistic, every norm and every cache write's arithmetic is fp32 in both.
//   embed_sinpos        x = table[token] + sinusoidal position vector (angle = p * base^(-2i/d), reduced in
//                       double so positions of any size keep an exact phase; sinf / cosf of the reduced angle)
//   layernorm_f32       (x - mean) / sqrt(var + eps) * w + b over fp32 rows (optionally gathered rows)
//   proj_norm_kv_write  the q and k projections RMS-normalised over the WHOLE projection (all heads at once),
//                       q scaled per head (softmax scale x temperature) into an fp32 buffer, k into the paged
//                       cache; v (4-token interleaved in its pages) blended with the values of an earlier layer (v <- (1 - lam) v + lam v0) or
//                       published as that v0, then into the paged cache
//   xielu               z > 0: ap z^2 + z/2;  z <= 0: an (expm1(z) - z) + z/2, ap = softplus(p), an = 1/2 + softplus(q)
//   residual_add_scaled x += m * y          residual_add_partials x += m * sum_s y_s (fp32 split-K partials)
#include "../common.h"

namespace lwc {
namespace {

template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  static LWC_DEVICE float ld(const bf16_t* p) { return bf2f(*p); }
  static LWC_DEVICE void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <> struct Elem<float> {
  static LWC_DEVICE float ld(const float* p) { return *p; }
  static LWC_DEVICE void st(float* p, float v) { *p = v; }
};

LWC_DEVICE float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename AT>
__global__ void embed_sinpos_kernel(const AT* __restrict__ table, const int* __restrict__ tokens,
                                    const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                    float* __restrict__ out, int d, int vocab) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const double p = (double)positions[t];
  const AT* row = table + (size_t)tok * d;
  float* o = out + (size_t)t * d;
  const double two_pi = 6.283185307179586476925286766559;
  for (int i = threadIdx.x; 2 * i < d; i += blockDim.x) {
    double a = p * inv_freq[i];
    a -= floor(a / two_pi) * two_pi;
    const float af = (float)a;
    o[2 * i] = Elem<AT>::ld(row + 2 * i) + sinf(af);
    if (2 * i + 1 < d) o[2 * i + 1] = Elem<AT>::ld(row + 2 * i + 1) + cosf(af);
  }
}

template <typename AT>
__global__ void layernorm_f32_kernel(const float* __restrict__ x, const long long* __restrict__ rows,
                                     const AT* __restrict__ w, const AT* __restrict__ b, AT* __restrict__ out, int d,
                                     float eps) {
  __shared__ float scratch[16];
  const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const float* xr = x + r * d;
  AT* o = out + (size_t)blockIdx.x * d;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) s += xr[i];
  const float mean = block_sum(s, scratch) / (float)d;
  float v = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float c = xr[i] - mean;
    v += c * c;
  }
  const float rstd = 1.0f / sqrtf(block_sum(v, scratch) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x)
    Elem<AT>::st(o + i, (xr[i] - mean) * rstd * Elem<AT>::ld(w + i) + Elem<AT>::ld(b + i));
}

// proj row t: [ q (nq = H*D) | k (nk = G*D) | v (nv = G*Dv) | ... ] with leading dimension ldp.
// vmode 0: v as projected; 1: publish v to v0 (fp32 [T, nv]); 2: v <- (1 - lam) v + lam v0.
template <typename AT>
__global__ void proj_norm_kv_write_kernel(const AT* __restrict__ proj, int ldp, const AT* __restrict__ wq,
                                          const AT* __restrict__ wk, const float* __restrict__ head_scale,
                                          const AT* __restrict__ lam_p, float* __restrict__ v0, int vmode,
                                          const int* __restrict__ slots, float* __restrict__ q_out,
                                          AT* __restrict__ k_cache, AT* __restrict__ v_cache, long long kb_stride,
                                          long long vb_stride, int block_size, int H, int D, int nk, int nv,
                                          float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int nq = H * D;
  const AT* pr = proj + (size_t)t * ldp;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const float q = Elem<AT>::ld(pr + i);
    sq += q * q;
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const float k = Elem<AT>::ld(pr + nq + i);
    sk += k * k;
  }
  const float rq = 1.0f / sqrtf(block_sum(sq, scratch) / (float)nq + eps);
  const float rk = 1.0f / sqrtf(block_sum(sk, scratch) / (float)nk + eps);
  float* qo = q_out + (size_t)t * nq;
  for (int i = threadIdx.x; i < nq; i += blockDim.x)
    qo[i] = Elem<AT>::ld(pr + i) * rq * Elem<AT>::ld(wq + i) * head_scale[i / D];
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  if (write) {
    AT* kc = k_cache + blk * kb_stride + off * nk;
    for (int i = threadIdx.x; i < nk; i += blockDim.x)
      Elem<AT>::st(kc + i, Elem<AT>::ld(pr + nq + i) * rk * Elem<AT>::ld(wk + i));
  }
  const float lam = vmode == 2 ? Elem<AT>::ld(lam_p) : 0.f;
  // V is 4-token interleaved: [block][offset / 4][column][offset % 4]
  AT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3);
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    float v = Elem<AT>::ld(pr + nq + nk + i);
    if (vmode == 1) v0[(size_t)t * nv + i] = v;
    if (vmode == 2) v = (1.0f - lam) * v + lam * v0[(size_t)t * nv + i];
    if (write) Elem<AT>::st(vc + 4 * i, v);
  }
}

template <typename AT>
__global__ void xielu_kernel(const AT* __restrict__ in, int ldi, const AT* __restrict__ pq, AT* __restrict__ out,
                             int ldo, int n, long long total) {
  const float ap = softplus(Elem<AT>::ld(pq)), an = 0.5f + softplus(Elem<AT>::ld(pq + 1));
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (long long)gridDim.x * blockDim.x) {
    const long long r = e / n;
    const int c = (int)(e - r * n);
    const float z = Elem<AT>::ld(in + r * ldi + c);
    const float y = z > 0.f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z;
    Elem<AT>::st(out + r * ldo + c, y);
  }
}

// bf16 rows whose width, leading dimensions and bases are multiples of 8 elements: 16 bytes per lane
__global__ void xielu_bf16x8_kernel(const bf16_t* __restrict__ in, int ldi, const bf16_t* __restrict__ pq,
                                    bf16_t* __restrict__ out, int ldo, int n8, long long total8) {
  const float ap = softplus(bf2f(pq[0])), an = 0.5f + softplus(bf2f(pq[1]));
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total8;
       e += (long long)gridDim.x * blockDim.x) {
    const long long r = e / n8;
    const int c = (int)(e - r * n8) * 8;
    float f[8];
    unpack8(*reinterpret_cast<const uint4v*>(in + r * ldi + c), f);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float z = f[k];
      f[k] = z > 0.f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z;
    }
    *reinterpret_cast<uint4v*>(out + r * ldo + c) = pack8(f);
  }
}

template <typename AT>
__global__ void residual_add_scaled_kernel(float* __restrict__ x, const AT* __restrict__ y, float m, long long total) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (long long)gridDim.x * blockDim.x)
    x[e] += m * Elem<AT>::ld(y + e);
}

// x += m * sum_s parts[s]  (fp32 partial products of a split-K GEMM)
__global__ void residual_add_partials_kernel(float* __restrict__ x, const float* __restrict__ parts, int S, float m,
                                             long long total) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (long long)gridDim.x * blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < S; ++s) acc += parts[(long long)s * total + e];
    x[e] += m * acc;
  }
}

// ---- 16-byte paths for bf16 activations (row widths, leading dimensions and bases multiples of 8 elements) ----
constexpr int kMaxChunks = 8;  // 8-element chunks a thread keeps in registers (rows up to 256 * 8 * 8 elements)

// LayerNorm of fp32 rows -> bf16: the row is read once (two float4 per chunk) and stays in registers.
__global__ void __launch_bounds__(256)
layernorm_f32_bf16x8_kernel(const float* __restrict__ x, const long long* __restrict__ rows, const bf16_t* __restrict__ w,
                            const bf16_t* __restrict__ b, bf16_t* __restrict__ out, int d, float eps) {
  __shared__ float scratch[16];
  const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const float* xr = x + r * d;
  const int nch = d >> 3;
  float v[kMaxChunks][8];
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    const int c = threadIdx.x + 256 * u;
    if (c < nch) {
      const float4v a0 = *reinterpret_cast<const float4v*>(xr + 8 * c), a1 = *reinterpret_cast<const float4v*>(xr + 8 * c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[u][e] = a0[e];
        v[u][4 + e] = a1[e];
        s += a0[e] + a1[e];
      }
    }
  }
  const float mean = block_sum(s, scratch) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    if (threadIdx.x + 256 * u < nch) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float c0 = v[u][e] - mean;
        q += c0 * c0;
      }
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(q, scratch) / (float)d + eps);
  bf16_t* o = out + (size_t)blockIdx.x * d;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    const int c = threadIdx.x + 256 * u;
    if (c < nch) {
      float wf[8], bf[8], y[8];
      unpack8(*reinterpret_cast<const uint4v*>(w + 8 * c), wf);
      unpack8(*reinterpret_cast<const uint4v*>(b + 8 * c), bf);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = (v[u][e] - mean) * rstd * wf[e] + bf[e];
      *reinterpret_cast<uint4v*>(o + 8 * c) = pack8(y);
    }
  }
}

// proj_norm_kv_write for bf16: the q | k | v part of the row is read once, 16 bytes per lane, and stays in registers.
__global__ void __launch_bounds__(256)
proj_norm_kv_write_bf16x8_kernel(const bf16_t* __restrict__ proj, int ldp, const bf16_t* __restrict__ wq,
                                 const bf16_t* __restrict__ wk, const float* __restrict__ head_scale,
                                 const bf16_t* __restrict__ lam_p, float* __restrict__ v0, int vmode,
                                 const int* __restrict__ slots, float* __restrict__ q_out, bf16_t* __restrict__ k_cache,
                                 bf16_t* __restrict__ v_cache, long long kb_stride, long long vb_stride, int block_size,
                                 int H, int D, int nk, int nv, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int nq = H * D, cq = nq >> 3, ck = nk >> 3, cv = nv >> 3, nch = cq + ck + cv;
  const bf16_t* pr = proj + (size_t)t * ldp;
  float v[kMaxChunks][8];
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    const int c = threadIdx.x + 256 * u;
    if (c < nch) {
      unpack8(*reinterpret_cast<const uint4v*>(pr + 8 * c), v[u]);
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[u][e] * v[u][e];
      if (c < cq) sq += ss;
      else if (c < cq + ck) sk += ss;
    }
  }
  const float rq = 1.0f / sqrtf(block_sum(sq, scratch) / (float)nq + eps);
  const float rk = 1.0f / sqrtf(block_sum(sk, scratch) / (float)nk + eps);
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  const float lam = vmode == 2 ? bf2f(*lam_p) : 0.f;
#pragma unroll
  for (int u = 0; u < kMaxChunks; ++u) {
    const int c = threadIdx.x + 256 * u;
    if (c >= nch) continue;
    if (c < cq) {
      float wf[8];
      unpack8(*reinterpret_cast<const uint4v*>(wq + 8 * c), wf);
      const float hs = head_scale[(8 * c) / D] * rq;  // (D is a multiple of 8: a chunk lies in one head)
      float* qo = q_out + (size_t)t * nq + 8 * c;
      *reinterpret_cast<float4v*>(qo) = float4v{v[u][0] * hs * wf[0], v[u][1] * hs * wf[1], v[u][2] * hs * wf[2], v[u][3] * hs * wf[3]};
      *reinterpret_cast<float4v*>(qo + 4) = float4v{v[u][4] * hs * wf[4], v[u][5] * hs * wf[5], v[u][6] * hs * wf[6], v[u][7] * hs * wf[7]};
    } else if (c < cq + ck) {
      if (write) {
        const int i = 8 * (c - cq);
        float wf[8], y[8];
        unpack8(*reinterpret_cast<const uint4v*>(wk + i), wf);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = v[u][e] * rk * wf[e];
        *reinterpret_cast<uint4v*>(k_cache + blk * kb_stride + off * nk + i) = pack8(y);
      }
    } else {
      const int i = 8 * (c - cq - ck);
      bf16_t* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float x = v[u][e];
        if (vmode == 1) v0[(size_t)t * nv + i + e] = x;
        if (vmode == 2) x = (1.0f - lam) * x + lam * v0[(size_t)t * nv + i + e];
        if (write) vc[4 * (i + e)] = f2bf(x);
      }
    }
  }
}

int grid_for(long long total, int block) {
  long long g = (total + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace
}  // namespace lwc

using namespace lwc;

#define R32_DISPATCH(f32, CALL_BF, CALL_F) \
  do {                                     \
    if (f32) { CALL_F; } else { CALL_BF; } \
  } while (0)

extern "C" {

int r32_embed_sinpos(const void* table, const int* tokens, const int* positions, const double* inv_freq, float* out,
                     int T, int d, int vocab, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  R32_DISPATCH(f32,
               (embed_sinpos_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)table, tokens, positions, inv_freq, out, d, vocab)),
               (embed_sinpos_kernel<float><<<T, 256, 0, s>>>((const float*)table, tokens, positions, inv_freq, out, d, vocab)));
  return (int)hipGetLastError();
}

int r32_layernorm(const float* x, const long long* rows, const void* w, const void* b, void* out, int T, int d,
                  float eps, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (!f32 && d % 8 == 0 && d <= 256 * 8 * kMaxChunks && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
      ((uintptr_t)b & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    layernorm_f32_bf16x8_kernel<<<T, 256, 0, s>>>(x, rows, (const bf16_t*)w, (const bf16_t*)b, (bf16_t*)out, d, eps);
    return (int)hipGetLastError();
  }
  R32_DISPATCH(f32,
               (layernorm_f32_kernel<bf16_t><<<T, 256, 0, s>>>(x, rows, (const bf16_t*)w, (const bf16_t*)b, (bf16_t*)out, d, eps)),
               (layernorm_f32_kernel<float><<<T, 256, 0, s>>>(x, rows, (const float*)w, (const float*)b, (float*)out, d, eps)));
  return (int)hipGetLastError();
}

int r32_proj_norm_kv_write(const void* proj, int ldp, const void* wq, const void* wk, const float* head_scale,
                           const void* lam, float* v0, int vmode, const int* slots, float* q_out, void* k_cache,
                           void* v_cache, long long kb_stride, long long vb_stride, int block_size, int T, int H, int D,
                           int nk, int nv, float eps, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (!f32 && D % 8 == 0 && nk % 8 == 0 && nv % 8 == 0 && ldp % 8 == 0 && (H * D + nk + nv) <= 256 * 8 * kMaxChunks &&
      kb_stride % 8 == 0 && ((uintptr_t)proj & 15) == 0 && ((uintptr_t)wq & 15) == 0 && ((uintptr_t)wk & 15) == 0 &&
      ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)q_out & 15) == 0) {
    proj_norm_kv_write_bf16x8_kernel<<<T, 256, 0, s>>>(
        (const bf16_t*)proj, ldp, (const bf16_t*)wq, (const bf16_t*)wk, head_scale, (const bf16_t*)lam, v0, vmode, slots, q_out,
        (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride, vb_stride, block_size, H, D, nk, nv, eps);
    return (int)hipGetLastError();
  }
  R32_DISPATCH(f32,
               (proj_norm_kv_write_kernel<bf16_t><<<T, 256, 0, s>>>(
                   (const bf16_t*)proj, ldp, (const bf16_t*)wq, (const bf16_t*)wk, head_scale, (const bf16_t*)lam, v0, vmode,
                   slots, q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride, vb_stride, block_size, H, D, nk, nv, eps)),
               (proj_norm_kv_write_kernel<float><<<T, 256, 0, s>>>(
                   (const float*)proj, ldp, (const float*)wq, (const float*)wk, head_scale, (const float*)lam, v0, vmode,
                   slots, q_out, (float*)k_cache, (float*)v_cache, kb_stride, vb_stride, block_size, H, D, nk, nv, eps)));
  return (int)hipGetLastError();
}

int r32_xielu(const void* in, int ldi, const void* pq, void* out, int ldo, int T, int n, int f32, hipStream_t s) {
  const long long total = (long long)T * n;
  if (total <= 0) return 0;
  if (!f32 && n % 8 == 0 && ldi % 8 == 0 && ldo % 8 == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    xielu_bf16x8_kernel<<<grid_for(total / 8, 256), 256, 0, s>>>((const bf16_t*)in, ldi, (const bf16_t*)pq, (bf16_t*)out, ldo,
                                                                 n / 8, total / 8);
    return (int)hipGetLastError();
  }
  const int g = grid_for(total, 256);
  R32_DISPATCH(f32,
               (xielu_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)in, ldi, (const bf16_t*)pq, (bf16_t*)out, ldo, n, total)),
               (xielu_kernel<float><<<g, 256, 0, s>>>((const float*)in, ldi, (const float*)pq, (float*)out, ldo, n, total)));
  return (int)hipGetLastError();
}

int r32_residual_add_scaled(float* x, const void* y, float m, long long total, int f32, hipStream_t s) {
  if (total <= 0) return 0;
  const int g = grid_for(total, 256);
  R32_DISPATCH(f32, (residual_add_scaled_kernel<bf16_t><<<g, 256, 0, s>>>(x, (const bf16_t*)y, m, total)),
               (residual_add_scaled_kernel<float><<<g, 256, 0, s>>>(x, (const float*)y, m, total)));
  return (int)hipGetLastError();
}

int r32_residual_add_partials(float* x, const float* parts, int S, float m, long long total, hipStream_t s) {
  if (total <= 0 || S <= 0) return 0;
  residual_add_partials_kernel<<<grid_for(total, 256), 256, 0, s>>>(x, parts, S, m, total);
  return (int)hipGetLastError();
}

}  // extern "C"

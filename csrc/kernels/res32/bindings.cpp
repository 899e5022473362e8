// torch bindings of the fp32-residual kernel set (llm_weighted_consensus_amd.ops._res32).
// Every op validates device, dtype and shape on the host, then launches on the caller's current HIP stream
// (capturable into a hipGraph).  Activation tensors are all bf16 or all fp32; the residual stream is fp32.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int r32_embed_sinpos(const void*, const int*, const int*, const double*, float*, int, int, int, int, hipStream_t);
int r32_layernorm(const float*, const long long*, const void*, const void*, void*, int, int, float, int, hipStream_t);
int r32_proj_norm_kv_write(const void*, int, const void*, const void*, const float*, const void*, float*, int,
                           const int*, float*, void*, void*, long long, long long, int, int, int, int, int, int, float,
                           int, hipStream_t);
int r32_xielu(const void*, int, const void*, void*, int, int, int, int, hipStream_t);
int r32_residual_add_scaled(float*, const void*, float, long long, int, hipStream_t);
int r32_residual_add_partials(float*, const float*, int, float, long long, hipStream_t);
int r32_window_attn(const float*, const void*, const void*, long long, long long, int, const int*, const int*, int,
                    const int*, int, const float*, const float*, int, void*, int, int, int, int, int, int, int,
                    hipStream_t);
int r32_window_attn_mfma_ok(int, int);
int r32_window_attn_mfma(const float*, const void*, const void*, long long, long long, int, const int*, const int*,
                         const int*, int, int, const int*, int, const float*, int, void*, int, int, int, int, int,
                         hipStream_t);
int r32_window_attn_decode_splits(int, int, int, int);
int r32_window_attn_decode(const float*, const void*, const void*, long long, long long, int, const int*, const int*, int,
                           const float*, int, float*, float*, int, int, void*, int, int, int, int, int, int, hipStream_t);
}

namespace {

using torch::Tensor;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

int act_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, ": expected a GPU tensor");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 || t.scalar_type() == torch::kFloat32, name, ": bf16 or fp32 expected");
  return t.scalar_type() == torch::kFloat32 ? 1 : 0;
}

void want(const Tensor& t, torch::ScalarType st, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == st && t.is_contiguous(), name, ": wrong device, dtype or layout");
}

void done(int rc, const char* name) { TORCH_CHECK(rc == 0, name, ": launch failed (", rc, ")"); }

// One layer's views of the paged pool: K [NB, BS, nk] token rows, V [NB, BS/4, nv, 4] 4-token interleaved.
void cache_layout(const Tensor& k, const Tensor& v, int& NB, int& BS, int& nk, int& nv, const char* name) {
  TORCH_CHECK(k.dim() == 3 && v.dim() == 4 && v.size(3) == 4, name, ": K [NB, BS, nk] and V [NB, BS/4, nv, 4] expected");
  NB = (int)k.size(0), BS = (int)k.size(1), nk = (int)k.size(2), nv = (int)v.size(2);
  TORCH_CHECK(BS % 4 == 0 && v.size(0) == NB && v.size(1) == BS / 4 && k.stride(2) == 1 && k.stride(1) == nk &&
                  v.stride(3) == 1 && v.stride(2) == 4 && v.stride(1) == 4 * (int64_t)nv, name, ": cache layout");
}

// rows of a 2-d tensor whose last dimension is dense; returns the leading dimension in elements
int row_stride(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1 && t.stride(0) >= t.size(1), name, ": rows must be dense");
  return (int)t.stride(0);
}

void embed_sinpos(Tensor table, Tensor tokens, Tensor positions, Tensor inv_freq, Tensor out) {
  const int f = act_f32(table, "embed_sinpos table");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_sinpos: table [V, d]");
  want(tokens, torch::kInt32, "embed_sinpos tokens");
  want(positions, torch::kInt32, "embed_sinpos positions");
  want(inv_freq, torch::kFloat64, "embed_sinpos inv_freq");
  want(out, torch::kFloat32, "embed_sinpos out");
  const int T = (int)tokens.numel(), d = (int)table.size(1);
  TORCH_CHECK(positions.numel() == T && out.dim() == 2 && out.size(0) == T && out.size(1) == d &&
                  inv_freq.numel() == (d + 1) / 2, "embed_sinpos: shapes disagree");
  done(r32_embed_sinpos(table.data_ptr(), tokens.data_ptr<int>(), positions.data_ptr<int>(), inv_freq.data_ptr<double>(),
                        out.data_ptr<float>(), T, d, (int)table.size(0), f, stream()), "embed_sinpos");
}

void layernorm(Tensor x, c10::optional<Tensor> rows, Tensor w, Tensor b, Tensor out, double eps) {
  want(x, torch::kFloat32, "layernorm x");
  const int f = act_f32(out, "layernorm out");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous() && w.is_contiguous() && b.is_contiguous(), "layernorm: layout");
  const int d = (int)x.size(1), T = (int)out.size(0);
  TORCH_CHECK(out.size(1) == d && w.numel() == d && b.numel() == d && w.scalar_type() == out.scalar_type() &&
                  b.scalar_type() == out.scalar_type() && w.is_cuda() && b.is_cuda(), "layernorm: shapes or dtypes disagree");
  const long long* rp = nullptr;
  if (rows.has_value()) {
    want(*rows, torch::kInt64, "layernorm rows");
    TORCH_CHECK(rows->numel() == T, "layernorm: one row index per output row");
    rp = (const long long*)rows->data_ptr<int64_t>();
  } else {
    TORCH_CHECK(x.size(0) == T, "layernorm: rows disagree");
  }
  done(r32_layernorm(x.data_ptr<float>(), rp, w.data_ptr(), b.data_ptr(), out.data_ptr(), T, d, (float)eps, f, stream()),
       "layernorm");
}

// proj [T, >= H*D + nk + nv] (row-dense); k_cache [NB, BS, nk], v_cache [NB, BS, nv] views of a pool (block strides
// taken from the views); q_out fp32 [T, H*D]; v0 fp32 [T, nv] when vmode != 0.
void proj_norm_kv_write(Tensor proj, Tensor wq, Tensor wk, Tensor head_scale, c10::optional<Tensor> lam,
                        c10::optional<Tensor> v0, int64_t vmode, Tensor slots, Tensor q_out, Tensor k_cache,
                        Tensor v_cache, int64_t H, int64_t D, double eps) {
  const int f = act_f32(proj, "proj_norm_kv_write proj");
  const int ldp = row_stride(proj, "proj_norm_kv_write proj");
  const int T = (int)proj.size(0);
  want(slots, torch::kInt32, "proj_norm_kv_write slots");
  want(q_out, torch::kFloat32, "proj_norm_kv_write q_out");
  want(head_scale, torch::kFloat32, "proj_norm_kv_write head_scale");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && k_cache.scalar_type() == proj.scalar_type() &&
                  v_cache.scalar_type() == proj.scalar_type(), "proj_norm_kv_write: caches of the activation dtype");
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "proj_norm_kv_write");
  const int nq = (int)(H * D);
  TORCH_CHECK(H > 0 && D > 0 && proj.size(1) >= nq + nk + nv && slots.numel() == T && q_out.numel() == (int64_t)T * nq &&
                  wq.numel() == nq && wk.numel() == nk && head_scale.numel() == H && wq.scalar_type() == proj.scalar_type() &&
                  wk.scalar_type() == proj.scalar_type() && wq.is_cuda() && wk.is_cuda() && wq.is_contiguous() &&
                  wk.is_contiguous(), "proj_norm_kv_write: shapes or dtypes disagree");
  TORCH_CHECK(vmode >= 0 && vmode <= 2, "proj_norm_kv_write: vmode");
  float* v0p = nullptr;
  const void* lp = nullptr;
  if (vmode != 0) {
    TORCH_CHECK(v0.has_value(), "proj_norm_kv_write: v0 buffer missing");
    want(*v0, torch::kFloat32, "proj_norm_kv_write v0");
    TORCH_CHECK(v0->numel() == (int64_t)T * nv, "proj_norm_kv_write: v0 [T, nv]");
    v0p = v0->data_ptr<float>();
  }
  if (vmode == 2) {
    TORCH_CHECK(lam.has_value() && lam->is_cuda() && lam->numel() == 1 && lam->scalar_type() == proj.scalar_type(),
                "proj_norm_kv_write: blend weight (one element of the activation dtype)");
    lp = lam->data_ptr();
  }
  done(r32_proj_norm_kv_write(proj.data_ptr(), ldp, wq.data_ptr(), wk.data_ptr(), head_scale.data_ptr<float>(), lp, v0p,
                              (int)vmode, slots.data_ptr<int>(), q_out.data_ptr<float>(), k_cache.data_ptr(),
                              v_cache.data_ptr(), (long long)k_cache.stride(0), (long long)v_cache.stride(0), BS, T, (int)H,
                              (int)D, nk, nv, (float)eps, f, stream()), "proj_norm_kv_write");
}

void xielu(Tensor in, Tensor pq, Tensor out) {
  const int f = act_f32(in, "xielu in");
  const int ldi = row_stride(in, "xielu in"), ldo = row_stride(out, "xielu out");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == in.scalar_type() && out.size(0) == in.size(0) && out.size(1) == in.size(1) &&
                  pq.is_cuda() && pq.numel() == 2 && pq.is_contiguous() && pq.scalar_type() == in.scalar_type(),
              "xielu: shapes or dtypes disagree");
  done(r32_xielu(in.data_ptr(), ldi, pq.data_ptr(), out.data_ptr(), ldo, (int)in.size(0), (int)in.size(1), f, stream()), "xielu");
}

void residual_add_scaled(Tensor x, Tensor y, double m) {
  want(x, torch::kFloat32, "residual_add_scaled x");
  const int f = act_f32(y, "residual_add_scaled y");
  TORCH_CHECK(y.is_contiguous() && y.numel() == x.numel(), "residual_add_scaled: shapes disagree");
  done(r32_residual_add_scaled(x.data_ptr<float>(), y.data_ptr(), (float)m, (long long)x.numel(), f, stream()),
       "residual_add_scaled");
}

void residual_add_partials(Tensor x, Tensor parts, double m) {
  want(x, torch::kFloat32, "residual_add_partials x");
  want(parts, torch::kFloat32, "residual_add_partials parts");
  TORCH_CHECK(parts.dim() >= 2 && parts.numel() == parts.size(0) * x.numel(), "residual_add_partials: parts [S, ...x]");
  done(r32_residual_add_partials(x.data_ptr<float>(), parts.data_ptr<float>(), (int)parts.size(0), (float)m,
                                 (long long)x.numel(), stream()), "residual_add_partials");
}

// q fp32 [T, H*D]; out [T, >= H*Dv] row-dense view of the cache dtype; block_tables [items, width] int32;
// cu_q: int32 [items + 1] for prompt portions, absent when row t is item t.
void window_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, c10::optional<Tensor> cu_q,
                 Tensor block_tables, Tensor r1, Tensor r2, int64_t window, Tensor out, int64_t H, int64_t G) {
  want(q, torch::kFloat32, "window_attn q");
  const int f = act_f32(k_cache, "window_attn k_cache");
  want(positions, torch::kInt32, "window_attn positions");
  want(block_tables, torch::kInt32, "window_attn block_tables");
  want(r1, torch::kFloat32, "window_attn r1");
  want(r2, torch::kFloat32, "window_attn r2");
  TORCH_CHECK(v_cache.is_cuda() && v_cache.scalar_type() == k_cache.scalar_type() && out.is_cuda() &&
                  out.scalar_type() == k_cache.scalar_type(), "window_attn: caches and out share a dtype");
  const int T = (int)positions.numel();
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "window_attn");
  TORCH_CHECK(G > 0 && H > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "window_attn: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  const int ldo = row_stride(out, "window_attn out");
  TORCH_CHECK(q.numel() == (int64_t)T * H * D && out.size(0) == T && out.size(1) == H * Dv && r1.numel() == H &&
                  r2.numel() == H && window >= 1 && block_tables.dim() == 2, "window_attn: shapes disagree");
  const int items = (int)block_tables.size(0), width = (int)block_tables.size(1);
  const int* cu = nullptr;
  if (cu_q.has_value()) {
    want(*cu_q, torch::kInt32, "window_attn cu_q");
    TORCH_CHECK(cu_q->numel() == items + 1, "window_attn: cu_q [items + 1]");
    cu = cu_q->data_ptr<int>();
  } else {
    TORCH_CHECK(items >= T, "window_attn: one table row per query row");
  }
  done(r32_window_attn(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                       (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), cu, items, block_tables.data_ptr<int>(),
                       width, r1.data_ptr<float>(), r2.data_ptr<float>(), (int)window, out.data_ptr(), ldo, T, (int)H, (int)G,
                       D, Dv, f, stream()), "window_attn");
}

bool window_attn_mfma_ok(int64_t D, int64_t Dv) { return r32_window_attn_mfma_ok((int)D, (int)Dv) != 0; }

// Prompt portions on the matrix cores: bf16 caches, q fp32 [T, H*D], bias fp32 [H, window] (the distance bias by
// i - j), cu_q / k_lens int32 per item (k_lens: the sequence's length after this step), max_q the longest portion.
// Positions ascend by one along each item's rows.
void window_attn_mfma(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, Tensor cu_q, Tensor k_lens,
                      int64_t max_q, Tensor block_tables, Tensor bias, int64_t window, Tensor out, int64_t H, int64_t G) {
  want(q, torch::kFloat32, "window_attn_mfma q");
  want(positions, torch::kInt32, "window_attn_mfma positions");
  want(block_tables, torch::kInt32, "window_attn_mfma block_tables");
  want(cu_q, torch::kInt32, "window_attn_mfma cu_q");
  want(k_lens, torch::kInt32, "window_attn_mfma k_lens");
  want(bias, torch::kFloat32, "window_attn_mfma bias");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && out.is_cuda() && k_cache.scalar_type() == torch::kBFloat16 &&
                  v_cache.scalar_type() == torch::kBFloat16 && out.scalar_type() == torch::kBFloat16,
              "window_attn_mfma: bf16 caches and out");
  const int T = (int)positions.numel();
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "window_attn_mfma");
  TORCH_CHECK(G > 0 && H > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "window_attn_mfma: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  TORCH_CHECK(r32_window_attn_mfma_ok(D, Dv), "window_attn_mfma: sizes not built");
  const int ldo = row_stride(out, "window_attn_mfma out");
  TORCH_CHECK(k_cache.stride(0) % 8 == 0 && v_cache.stride(0) % 8 == 0 && ((uintptr_t)k_cache.data_ptr() & 15) == 0 &&
                  ((uintptr_t)v_cache.data_ptr() & 15) == 0, "window_attn_mfma: cache alignment");
  const int items = (int)block_tables.size(0);
  TORCH_CHECK(block_tables.dim() == 2 && cu_q.numel() == items + 1 && k_lens.numel() == items && max_q >= 1 &&
                  q.numel() == (int64_t)T * H * D && out.size(0) == T && out.size(1) == H * Dv && window >= 1 &&
                  bias.numel() == H * window, "window_attn_mfma: shapes disagree");
  done(r32_window_attn_mfma(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                            (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), cu_q.data_ptr<int>(),
                            k_lens.data_ptr<int>(), items, (int)max_q, block_tables.data_ptr<int>(),
                            (int)block_tables.size(1), bias.data_ptr<float>(), (int)window, out.data_ptr(), ldo, (int)H, (int)G,
                            D, Dv, stream()), "window_attn_mfma");
}

// One new token per sequence on the matrix cores (bf16 caches): row b reads table row b, its key range ends at
// positions[b].  max_keys: a host-side upper bound of the keys a row sees (min(window, longest context)).
void window_attn_decode(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, Tensor block_tables, Tensor bias,
                        int64_t window, int64_t max_keys, Tensor out, int64_t H, int64_t G) {
  want(q, torch::kFloat32, "window_attn_decode q");
  want(positions, torch::kInt32, "window_attn_decode positions");
  want(block_tables, torch::kInt32, "window_attn_decode block_tables");
  want(bias, torch::kFloat32, "window_attn_decode bias");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && out.is_cuda() && k_cache.scalar_type() == torch::kBFloat16 &&
                  v_cache.scalar_type() == torch::kBFloat16 && out.scalar_type() == torch::kBFloat16,
              "window_attn_decode: bf16 caches and out");
  const int B = (int)positions.numel();
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "window_attn_decode");
  TORCH_CHECK(G > 0 && H > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "window_attn_decode: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  TORCH_CHECK(r32_window_attn_mfma_ok(D, Dv), "window_attn_decode: sizes not built");
  const int ldo = row_stride(out, "window_attn_decode out");
  TORCH_CHECK(k_cache.stride(0) % 8 == 0 && v_cache.stride(0) % 8 == 0 && ((uintptr_t)k_cache.data_ptr() & 15) == 0 &&
                  ((uintptr_t)v_cache.data_ptr() & 15) == 0, "window_attn_decode: cache alignment");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= B && q.numel() == (int64_t)B * H * D && out.size(0) == B &&
                  out.size(1) == H * Dv && window >= 1 && max_keys >= 1 && bias.numel() == H * window,
              "window_attn_decode: shapes disagree");
  const int S = r32_window_attn_decode_splits(B, (int)G, (int)(H / G), (int)max_keys);
  auto part = torch::empty({(int64_t)B * H * S * (Dv + 2)}, q.options());
  float* po = part.data_ptr<float>();
  done(r32_window_attn_decode(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                              (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), block_tables.data_ptr<int>(),
                              (int)block_tables.size(1), bias.data_ptr<float>(), (int)window, po, po + (int64_t)B * H * S * Dv, S,
                              (int)max_keys, out.data_ptr(), ldo, B, (int)H, (int)G, D, Dv, stream()), "window_attn_decode");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "llm_weighted_consensus_amd fp32-residual kernel set (gfx950)";
  m.def("embed_sinpos", &embed_sinpos);
  m.def("layernorm", &layernorm);
  m.def("proj_norm_kv_write", &proj_norm_kv_write);
  m.def("xielu", &xielu);
  m.def("residual_add_scaled", &residual_add_scaled);
  m.def("residual_add_partials", &residual_add_partials);
  m.def("window_attn", &window_attn);
  m.def("window_attn_mfma", &window_attn_mfma);
  m.def("window_attn_mfma_ok", &window_attn_mfma_ok);
  m.def("window_attn_decode", &window_attn_decode);
}

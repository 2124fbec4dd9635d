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
                    const int*, int, const float*, const float*, const float*, int, int, void*, int, int, int, int, int, int, int,
                    hipStream_t);
int r32_window_attn_mfma_ok(int, int);
int r32_window_attn_mfma(const float*, const void*, const void*, long long, long long, int, const int*, const int*,
                         const int*, int, int, const int*, int, const float*, const float*, int, int, void*, int, int, int, int, int,
                         hipStream_t);
int r32_window_attn_decode_ok(int, int, int);
int r32_window_attn_decode_splits(int, int, int, int, int);
int r32_window_attn_decode(const float*, const void*, const void*, long long, long long, int, const int*, const int*, int,
                           const float*, const float*, int, int, float*, float*, int, int, void*, int, int, int, int, int, int, int,
                           hipStream_t);
int r32_conv_hist(const void*, int, const float*, int, int, float*, long long, const int*, const int*, const int*,
                  const int*, void*, int, void*, int, int, int, int, int, int, int, hipStream_t);
int r32_conv_hist_update(const void*, int, float*, long long, const int*, const int*, int, int, int, int, hipStream_t);
int r32_delta_rule_max_dim();
int r32_delta_rule(float*, int, const void*, int, int, int, const float*, const float*, float*, float*, long long, const int*,
                   const int*, const int*, float*, int, int, int, int, int, int, int, int, hipStream_t);
int r32_head_norm_gate(const float*, int, const void*, int, const float*, void*, int, int, int, int, float, int, int,
                       hipStream_t);
int r32_embed_rows(const void*, const int*, float*, int, int, int, float, int, hipStream_t);
int r32_head_norm_kv_write(const void*, int, int, int, const int*, const int*, float*, void*, void*, long long, long long,
                           int, int, int, int, int, int, float, float, float, int, int, hipStream_t);
int r32_gate_mul(void*, int, const void*, int, int, int, int, int, hipStream_t);
int r32_gated_norm_residual(float*, const void*, int, const void*, int, const float*, void*, const float*, int, int, float,
                            int, int, hipStream_t);
int r32_latent_expand_write(const void*, int, const void*, int, int, const long long*, void*, void*, long long, long long,
                            int, int, int, int, int, int, int, int, int, hipStream_t);
int r32_rmsnorm_rows(const float*, const long long*, const float*, void*, int, int, float, int, hipStream_t);
int r32_gelu_mul_rows(const void*, int, const void*, int, int, const int*, int, void*, int, int, int, hipStream_t);
int r32_stack_mix(const float*, long long, const float*, int, float*, long long, hipStream_t);
int r32_router_max_outputs();
int r32_router(const float*, const float*, const float*, int, int, int, int, int, int*, float*, int*, int*, int*, int*, int*,
               int*, hipStream_t);
int r32_expert_rows(const void*, int, const int*, const int*, const int*, int, const void*, const void*, float*, int, int,
                    int, int, hipStream_t);
int r32_moe_combine(const void*, int, const int*, const float*, const void*, int, int, int, float*, int, const void*, int, int,
                    hipStream_t);
int r32_latent_kv_write(const void*, int, int, int, int, const float*, const float*, const float*, float, const int*,
                        const int*, void*, int, void*, void*, long long, long long, int, int, int, float, int, int,
                        hipStream_t);
int r32_latent_q_rows(const void*, int, int, int, const float*, int, const float*, float, float, const int*, float*, int, int,
                      int, int, hipStream_t);
int r32_retention_max_dim();
int r32_retention_prep(const void*, int, int, const float*, float, const int*, float*, int, int, int, int, float, int,
                       hipStream_t);
int r32_retention(const float*, const void*, int, const float*, float*, long long, const int*, const int*, const int*, float*,
                  int, int, int, int, int, int, hipStream_t);
int r32_glu(const void*, int, void*, int, int, int, int, float, float, int, hipStream_t);
int r32_gelu(const void*, int, void*, int, int, int, int, hipStream_t);
int r32_rot_kv_write(const void*, int, const float*, const float*, const float*, float, int, const float*, const int*,
                     const int*, float*, void*, void*, long long, long long, int, int, int, int, int, int, float, float, int,
                     hipStream_t);
int r32_head_gate_unrotate(const void*, int, const void*, int, const float*, const int*, void*, int, int, int, int, float,
                           int, hipStream_t);
int r32_add_rmsnorm(float*, const void*, int, const float*, void*, int, int, int, float, int, hipStream_t);
int r32_chan_rule_max_dim();
int r32_chan_rule(const void*, int, int, float*, int, const void*, int, int, const float*, const float*, float, const void*,
                  int, int, float*, float*, float*, long long, const int*, const int*, const int*, float*, int, int, int, int,
                  int, int, int, int, int, hipStream_t);
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

void want_dev(const Tensor& t, torch::ScalarType st, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == st, name, ": wrong device or dtype");
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
// sink: fp32 [H], exp(sink_h) joins head h's softmax denominator (no key, no value), or absent.
void window_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, c10::optional<Tensor> cu_q,
                 Tensor block_tables, Tensor r1, Tensor r2, int64_t window, Tensor out, int64_t H, int64_t G,
                 c10::optional<Tensor> sink, int64_t chunk) {
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
  const float* sk = nullptr;
  if (sink.has_value()) {
    want(*sink, torch::kFloat32, "window_attn sink");
    TORCH_CHECK(sink->numel() == H, "window_attn: sink [H]");
    sk = sink->data_ptr<float>();
  }
  done(r32_window_attn(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                       (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), cu, items, block_tables.data_ptr<int>(),
                       width, r1.data_ptr<float>(), r2.data_ptr<float>(), sk, (int)window, (int)chunk, out.data_ptr(), ldo, T, (int)H, (int)G,
                       D, Dv, f, stream()), "window_attn");
}

bool window_attn_mfma_ok(int64_t D, int64_t Dv) { return r32_window_attn_mfma_ok((int)D, (int)Dv) != 0; }
bool window_attn_decode_ok(int64_t D, int64_t Dv, bool values_in_keys) {
  return r32_window_attn_decode_ok((int)D, (int)Dv, values_in_keys ? 1 : 0) != 0;
}

const float* sink_ptr(const c10::optional<Tensor>& sink, int64_t H, const char* name) {
  if (!sink.has_value()) return nullptr;
  want(*sink, torch::kFloat32, name);
  TORCH_CHECK(sink->numel() == H, name, ": sink [H]");
  return sink->data_ptr<float>();
}

// Prompt portions on the matrix cores: bf16 caches, q fp32 [T, H*D], bias fp32 [H, window] (the distance bias by
// i - j), cu_q / k_lens int32 per item (k_lens: the sequence's length after this step), max_q the longest portion.
// Positions ascend by one along each item's rows.
void window_attn_mfma(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, Tensor cu_q, Tensor k_lens,
                      int64_t max_q, Tensor block_tables, c10::optional<Tensor> bias, int64_t window, Tensor out, int64_t H,
                      int64_t G, c10::optional<Tensor> sink, int64_t chunk) {
  want(q, torch::kFloat32, "window_attn_mfma q");
  want(positions, torch::kInt32, "window_attn_mfma positions");
  want(block_tables, torch::kInt32, "window_attn_mfma block_tables");
  want(cu_q, torch::kInt32, "window_attn_mfma cu_q");
  want(k_lens, torch::kInt32, "window_attn_mfma k_lens");
  if (bias.has_value()) want(*bias, torch::kFloat32, "window_attn_mfma bias");
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
                  (!bias.has_value() || bias->numel() == H * window), "window_attn_mfma: shapes disagree");
  done(r32_window_attn_mfma(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                            (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), cu_q.data_ptr<int>(),
                            k_lens.data_ptr<int>(), items, (int)max_q, block_tables.data_ptr<int>(),
                            (int)block_tables.size(1), bias.has_value() ? bias->data_ptr<float>() : nullptr,
                            sink_ptr(sink, H, "window_attn_mfma"), (int)window, (int)chunk, out.data_ptr(), ldo, (int)H, (int)G, D, Dv,
                            stream()), "window_attn_mfma");
}

// One new token per sequence on the matrix cores (bf16 caches): row b reads table row b, its key range ends at
// positions[b].  max_keys: a host-side upper bound of the keys a row sees (min(window, longest context)).
void window_attn_decode(Tensor q, Tensor k_cache, Tensor v_cache, Tensor positions, Tensor block_tables,
                        c10::optional<Tensor> bias, int64_t window, int64_t max_keys, Tensor out, int64_t H, int64_t G,
                        c10::optional<Tensor> sink, bool values_in_keys, int64_t chunk) {
  want(q, torch::kFloat32, "window_attn_decode q");
  want(positions, torch::kInt32, "window_attn_decode positions");
  want(block_tables, torch::kInt32, "window_attn_decode block_tables");
  if (bias.has_value()) want(*bias, torch::kFloat32, "window_attn_decode bias");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && out.is_cuda() && k_cache.scalar_type() == torch::kBFloat16 &&
                  v_cache.scalar_type() == torch::kBFloat16 && out.scalar_type() == torch::kBFloat16,
              "window_attn_decode: bf16 caches and out");
  const int B = (int)positions.numel();
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "window_attn_decode");
  TORCH_CHECK(G > 0 && H > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "window_attn_decode: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  TORCH_CHECK(r32_window_attn_decode_ok(D, Dv, values_in_keys ? 1 : 0), "window_attn_decode: sizes not built");
  const int ldo = row_stride(out, "window_attn_decode out");
  TORCH_CHECK(k_cache.stride(0) % 8 == 0 && v_cache.stride(0) % 8 == 0 && ((uintptr_t)k_cache.data_ptr() & 15) == 0 &&
                  ((uintptr_t)v_cache.data_ptr() & 15) == 0, "window_attn_decode: cache alignment");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= B && q.numel() == (int64_t)B * H * D && out.size(0) == B &&
                  out.size(1) == H * Dv && window >= 1 && max_keys >= 1 && (!bias.has_value() || bias->numel() == H * window),
              "window_attn_decode: shapes disagree");
  const int S = r32_window_attn_decode_splits(B, (int)G, (int)(H / G), (int)max_keys, D);
  auto part = torch::empty({(int64_t)B * H * S * (Dv + 2)}, q.options());
  float* po = part.data_ptr<float>();
  done(r32_window_attn_decode(q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                              (long long)v_cache.stride(0), BS, positions.data_ptr<int>(), block_tables.data_ptr<int>(),
                              (int)block_tables.size(1), bias.has_value() ? bias->data_ptr<float>() : nullptr,
                              sink_ptr(sink, H, "window_attn_decode"), (int)window, (int)chunk, po, po + (int64_t)B * H * S * Dv, S,
                              (int)max_keys, out.data_ptr(), ldo, B, (int)H, (int)G, D, Dv, values_in_keys ? 1 : 0, stream()),
       "window_attn_decode");
}


// ---------------------------------------------------------------- recurrent state, gated layers, routed experts
// Items: rows [cu[i], cu[i+1]) of one sequence at consecutive positions, with state slot item_slot[i].
struct Items {
  const int *row_item, *cu, *slot, *pos;
  int T, n;
};

Items items_of(const Tensor& row_item, const Tensor& cu, const Tensor& item_slot, const Tensor& positions, int64_t slots,
               const char* name) {
  want(row_item, torch::kInt32, name);
  want(cu, torch::kInt32, name);
  want(item_slot, torch::kInt32, name);
  want(positions, torch::kInt32, name);
  const int T = (int)positions.numel(), n = (int)item_slot.numel();
  TORCH_CHECK(row_item.numel() == T && cu.numel() == n + 1 && slots > 0, name, ": item tables disagree");
  return {row_item.data_ptr<int>(), cu.data_ptr<int>(), item_slot.data_ptr<int>(), positions.data_ptr<int>(), T, n};
}

// hist fp32 [slots, taps - 1, C] (a strided view of a slot pool: slot stride taken from the view)
long long hist_layout(const Tensor& hist, int taps, int C, const char* name) {
  want_dev(hist, torch::kFloat32, name);
  TORCH_CHECK(hist.dim() == 3 && hist.size(1) == taps - 1 && hist.size(2) == C && hist.stride(2) == 1 &&
                  (taps == 1 || hist.stride(1) == C), name, ": history [slots, taps - 1, C]");
  return (long long)hist.stride(0);
}

// mode 0: out = x + conv(x), out2 (optional) = x in out's dtype; mode 1: out = silu(conv(x)); mode 2: out = conv(x).
// w fp32 [C, taps].
// advance: every item is ONE row (a decode step) and the kernel also moves the slots' histories on.
void conv_hist(Tensor x, Tensor w, Tensor hist, Tensor row_item, Tensor cu, Tensor item_slot, Tensor positions, Tensor out,
               c10::optional<Tensor> out2, int64_t mode, bool advance) {
  const int fi = act_f32(x, "conv_hist x"), fo = act_f32(out, "conv_hist out");
  const int ldx = row_stride(x, "conv_hist x"), ldo = row_stride(out, "conv_hist out");
  want_dev(w, torch::kFloat32, "conv_hist w");  // [C, taps], any strides (tap-major storage takes the 16-byte path)
  const int C = (int)x.size(1), taps = (int)w.size(1);
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && out.size(0) == x.size(0) && out.size(1) == C, "conv_hist: shapes disagree");
  const long long ss = hist_layout(hist, taps, C, "conv_hist hist");
  Items it = items_of(row_item, cu, item_slot, positions, hist.size(0), "conv_hist items");
  TORCH_CHECK(it.T == x.size(0), "conv_hist: one position per row");
  TORCH_CHECK(!advance || it.n == it.T, "conv_hist: the fused history update wants items of one row");
  void* o2 = nullptr;
  int ldo2 = 0;
  if (out2.has_value()) {
    TORCH_CHECK(mode == 0 && out2->scalar_type() == out.scalar_type() && out2->is_cuda() && out2->size(0) == x.size(0) &&
                    out2->size(1) == C, "conv_hist: out2");
    ldo2 = row_stride(*out2, "conv_hist out2");
    o2 = out2->data_ptr();
  }
  done(r32_conv_hist(x.data_ptr(), ldx, w.data_ptr<float>(), (int)w.stride(0), (int)w.stride(1), hist.data_ptr<float>(), ss,
                     it.row_item, it.cu, it.slot, it.pos,
                     out.data_ptr(), ldo, o2, ldo2, it.T, C, taps, (int)mode, fi | (fo << 1), advance ? 1 : 0, stream()), "conv_hist");
}

void conv_hist_update(Tensor x, Tensor hist, Tensor cu, Tensor item_slot, int64_t taps) {
  const int fi = act_f32(x, "conv_hist_update x");
  const int ldx = row_stride(x, "conv_hist_update x");
  const int C = (int)x.size(1);
  want(cu, torch::kInt32, "conv_hist_update cu");
  want(item_slot, torch::kInt32, "conv_hist_update item_slot");
  TORCH_CHECK(cu.numel() == item_slot.numel() + 1, "conv_hist_update: cu [items + 1]");
  if (taps <= 1) return;
  const long long ss = hist_layout(hist, (int)taps, C, "conv_hist_update hist");
  done(r32_conv_hist_update(x.data_ptr(), ldx, hist.data_ptr<float>(), ss, cu.data_ptr<int>(), item_slot.data_ptr<int>(),
                            (int)item_slot.numel(), C, (int)taps, fi, stream()), "conv_hist_update");
}

int64_t delta_rule_max_dim() { return r32_delta_rule_max_dim(); }

// qkv fp32 [T, 2 G D + H Dv] (its q and k columns are normalised in place); ba [T, ...] with beta logits at b_off and decay inputs at a_off (H columns each);
// state fp32 [slots, H, D, Dv] view; out fp32 [T, H Dv]
void delta_rule(Tensor qkv, Tensor ba, int64_t b_off, int64_t a_off, Tensor A_log, Tensor dt_bias, Tensor state, Tensor cu,
                Tensor item_slot, Tensor positions, Tensor out, int64_t H, int64_t G) {
  want_dev(qkv, torch::kFloat32, "delta_rule qkv");
  const int ldq = row_stride(qkv, "delta_rule qkv");
  const int f = act_f32(ba, "delta_rule ba");
  const int ldb = row_stride(ba, "delta_rule ba");
  want(A_log, torch::kFloat32, "delta_rule A_log");
  want(dt_bias, torch::kFloat32, "delta_rule dt_bias");
  want_dev(state, torch::kFloat32, "delta_rule state");
  want(cu, torch::kInt32, "delta_rule cu");
  want(item_slot, torch::kInt32, "delta_rule item_slot");
  want(positions, torch::kInt32, "delta_rule positions");
  want_dev(out, torch::kFloat32, "delta_rule out");
  const int ldo = row_stride(out, "delta_rule out");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.stride(3) == 1 && state.stride(2) == state.size(3) &&
                  state.stride(1) == state.size(2) * state.size(3), "delta_rule: state [slots, H, D, Dv]");
  const int D = (int)state.size(2), Dv = (int)state.size(3), T = (int)qkv.size(0);
  TORCH_CHECK(G > 0 && H % G == 0 && qkv.size(1) == 2 * G * D + H * Dv && out.size(0) == T && out.size(1) == H * Dv &&
                  ba.size(0) == T && b_off >= 0 && a_off >= 0 && b_off + H <= ba.size(1) && a_off + H <= ba.size(1) &&
                  A_log.numel() == H && dt_bias.numel() == H && positions.numel() == T && cu.numel() == item_slot.numel() + 1 &&
                  D <= r32_delta_rule_max_dim(), "delta_rule: shapes disagree");
  Tensor bg = torch::empty({T, 2 * H + G}, qkv.options());
  done(r32_delta_rule(qkv.data_ptr<float>(), ldq, ba.data_ptr(), ldb, (int)b_off, (int)a_off, A_log.data_ptr<float>(),
                      dt_bias.data_ptr<float>(), bg.data_ptr<float>(), state.data_ptr<float>(), (long long)state.stride(0),
                      cu.data_ptr<int>(), item_slot.data_ptr<int>(), positions.data_ptr<int>(), out.data_ptr<float>(), ldo, T,
                      (int)item_slot.numel(), (int)H, (int)G, D, Dv, f, stream()), "delta_rule");
}

// o fp32 [T, H Dv]; gate (mode 1 silu, 2 sigmoid; 0: unused) and out of the activation dtype; w fp32 [Dv] or absent
void head_norm_gate(Tensor o, c10::optional<Tensor> gate, c10::optional<Tensor> w, Tensor out, int64_t H, double eps,
                    int64_t mode) {
  want_dev(o, torch::kFloat32, "head_norm_gate o");
  const int ldi = row_stride(o, "head_norm_gate o"), ldo = row_stride(out, "head_norm_gate out");
  const int f = act_f32(out, "head_norm_gate out");
  const int T = (int)o.size(0);
  TORCH_CHECK(H > 0 && o.size(1) % H == 0 && out.size(0) == T && out.size(1) == o.size(1), "head_norm_gate: shapes");
  const int Dv = (int)(o.size(1) / H);
  const void* gp = nullptr;
  int ldg = 0;
  if (mode != 0) {
    TORCH_CHECK(gate.has_value() && gate->is_cuda() && gate->scalar_type() == out.scalar_type() && gate->size(0) == T &&
                    gate->size(1) == o.size(1), "head_norm_gate: gate");
    ldg = row_stride(*gate, "head_norm_gate gate");
    gp = gate->data_ptr();
  }
  const float* wp = nullptr;
  if (w.has_value()) {
    want(*w, torch::kFloat32, "head_norm_gate w");
    TORCH_CHECK(w->numel() == Dv, "head_norm_gate: w [Dv]");
    wp = w->data_ptr<float>();
  }
  done(r32_head_norm_gate(o.data_ptr<float>(), ldi, gp, ldg, wp, out.data_ptr(), ldo, T, (int)H, Dv, (float)eps, (int)mode, f,
                          stream()), "head_norm_gate");
}

void embed_rows(Tensor table, Tensor tokens, Tensor out, double scale) {
  const int f = act_f32(table, "embed_rows table");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_rows: table [V, d]");
  want(tokens, torch::kInt32, "embed_rows tokens");
  want(out, torch::kFloat32, "embed_rows out");
  const int T = (int)tokens.numel(), d = (int)table.size(1);
  TORCH_CHECK(out.numel() == (int64_t)T * d, "embed_rows: out [T, d]");
  done(r32_embed_rows(table.data_ptr(), tokens.data_ptr<int>(), out.data_ptr<float>(), T, d, (int)table.size(0), (float)scale, f,
                      stream()), "embed_rows");
}

// proj [T, ...] row-dense: q at column 0 (H*D), k at k_off (G*D), values at v_off (G*Dv; v_off == k_off: the keys as
// projected are the values)
void head_norm_kv_write(Tensor proj, int64_t k_off, int64_t v_off, Tensor positions, Tensor slots, Tensor q_out,
                        Tensor k_cache, Tensor v_cache, int64_t H, int64_t G, double eps, double scale, double coef,
                        int64_t every) {
  const int f = act_f32(proj, "head_norm_kv_write proj");
  const int ldp = row_stride(proj, "head_norm_kv_write proj");
  const int T = (int)proj.size(0);
  want(positions, torch::kInt32, "head_norm_kv_write positions");
  want(slots, torch::kInt32, "head_norm_kv_write slots");
  want(q_out, torch::kFloat32, "head_norm_kv_write q_out");
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() && k_cache.scalar_type() == proj.scalar_type() &&
                  v_cache.scalar_type() == proj.scalar_type(), "head_norm_kv_write: caches of the activation dtype");
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "head_norm_kv_write");
  TORCH_CHECK(G > 0 && H > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "head_norm_kv_write: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  TORCH_CHECK(positions.numel() == T && slots.numel() == T && q_out.numel() == (int64_t)T * H * D && k_off >= H * D &&
                  k_off + nk <= proj.size(1) && v_off >= 0 && v_off + nv <= proj.size(1) && every >= 0,
              "head_norm_kv_write: shapes disagree");
  done(r32_head_norm_kv_write(proj.data_ptr(), ldp, (int)k_off, (int)v_off, positions.data_ptr<int>(), slots.data_ptr<int>(),
                              q_out.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                              (long long)v_cache.stride(0), BS, T, (int)H, (int)G, D, Dv, (float)eps, (float)scale, (float)coef,
                              (int)every, f, stream()), "head_norm_kv_write");
}

void gate_mul(Tensor a, Tensor g, int64_t mode) {
  const int f = act_f32(a, "gate_mul a");
  const int lda = row_stride(a, "gate_mul a"), ldg = row_stride(g, "gate_mul g");
  TORCH_CHECK(g.is_cuda() && g.scalar_type() == a.scalar_type() && g.size(0) == a.size(0) && g.size(1) == a.size(1) &&
                  (mode == 0 || mode == 1), "gate_mul: shapes or dtypes disagree");
  done(r32_gate_mul(a.data_ptr(), lda, g.data_ptr(), ldg, (int)a.size(0), (int)a.size(1), (int)mode, f, stream()), "gate_mul");
}

// w_next (fp32 [d]): x_cast receives the NEXT sublayer's input norm of the new x, x / rms(x) * w_next, instead of a copy
void gated_norm_residual(Tensor x, Tensor y, c10::optional<Tensor> r, Tensor w, c10::optional<Tensor> x_cast, double eps,
                         c10::optional<Tensor> w_next) {
  want(x, torch::kFloat32, "gated_norm_residual x");
  want(w, torch::kFloat32, "gated_norm_residual w");
  const int fy = act_f32(y, "gated_norm_residual y");
  const int ldy = row_stride(y, "gated_norm_residual y");
  const int T = (int)x.size(0), d = (int)x.size(1);
  TORCH_CHECK(x.dim() == 2 && y.size(0) == T && y.size(1) == d && w.numel() == d, "gated_norm_residual: shapes disagree");
  const void* rp = nullptr;
  int ldr = 0, fr = 0;
  if (r.has_value()) {
    fr = act_f32(*r, "gated_norm_residual r");
    ldr = row_stride(*r, "gated_norm_residual r");
    TORCH_CHECK(r->size(0) == T && r->size(1) == d, "gated_norm_residual: gate logits [T, d]");
    rp = r->data_ptr();
  }
  void* xc = nullptr;
  if (x_cast.has_value()) {
    want(*x_cast, torch::kBFloat16, "gated_norm_residual x_cast");
    TORCH_CHECK(x_cast->numel() == x.numel(), "gated_norm_residual: x_cast [T, d]");
    xc = x_cast->data_ptr();
  }
  const float* wn = nullptr;
  if (w_next.has_value()) {
    want(*w_next, torch::kFloat32, "gated_norm_residual w_next");
    TORCH_CHECK(w_next->numel() == d && xc != nullptr, "gated_norm_residual: w_next [d] needs x_cast");
    wn = w_next->data_ptr<float>();
  }
  done(r32_gated_norm_residual(x.data_ptr<float>(), y.data_ptr(), ldy, rp, ldr, w.data_ptr<float>(), xc, wn, T, d, (float)eps,
                               fy, fr, stream()), "gated_norm_residual");
}

void rmsnorm_rows(Tensor x, c10::optional<Tensor> rows, Tensor w, Tensor out, double eps) {
  want(x, torch::kFloat32, "rmsnorm_rows x");
  want(w, torch::kFloat32, "rmsnorm_rows w");
  const int f = act_f32(out, "rmsnorm_rows out");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous() && out.size(1) == x.size(1) && w.numel() == x.size(1),
              "rmsnorm_rows: shapes disagree");
  const long long* rp = nullptr;
  if (rows.has_value()) {
    want(*rows, torch::kInt64, "rmsnorm_rows rows");
    TORCH_CHECK(rows->numel() == out.size(0), "rmsnorm_rows: one row index per output row");
    rp = (const long long*)rows->data_ptr<int64_t>();
  } else {
    TORCH_CHECK(x.size(0) == out.size(0), "rmsnorm_rows: rows disagree");
  }
  done(r32_rmsnorm_rows(x.data_ptr<float>(), rp, w.data_ptr<float>(), out.data_ptr(), (int)out.size(0), (int)x.size(1),
                        (float)eps, f, stream()), "rmsnorm_rows");
}

// out [T, n] = gelu_tanh(z [T, n]) * table[tokens[t]][off : off + n]
void gelu_mul_rows(Tensor z, Tensor table, int64_t off, Tensor tokens, Tensor out) {
  const int f = act_f32(z, "gelu_mul_rows z");
  const int ldz = row_stride(z, "gelu_mul_rows z"), ldt = row_stride(table, "gelu_mul_rows table");
  want(tokens, torch::kInt32, "gelu_mul_rows tokens");
  const int T = (int)z.size(0), n = (int)z.size(1);
  TORCH_CHECK(table.is_cuda() && table.scalar_type() == z.scalar_type() && out.is_cuda() && out.scalar_type() == z.scalar_type() &&
                  out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == n && tokens.numel() == T && off >= 0 &&
                  off + n <= table.size(1), "gelu_mul_rows: shapes or dtypes disagree");
  done(r32_gelu_mul_rows(z.data_ptr(), ldz, table.data_ptr(), ldt, (int)off, tokens.data_ptr<int>(), (int)table.size(0),
                         out.data_ptr(), T, n, f, stream()), "gelu_mul_rows");
}

// out = sum_{j < n} coef[j] * X[j]; X fp32 [>= n, ...] contiguous, out one plane of it (it may be a plane of X
// beyond the first n)
void stack_mix(Tensor X, Tensor coef, int64_t n, Tensor out) {
  want(X, torch::kFloat32, "stack_mix X");
  want(coef, torch::kFloat32, "stack_mix coef");
  want(out, torch::kFloat32, "stack_mix out");
  TORCH_CHECK(X.dim() >= 2 && n >= 1 && n <= X.size(0) && coef.numel() >= n && out.numel() * X.size(0) == X.numel(),
              "stack_mix: shapes disagree");
  done(r32_stack_mix(X.data_ptr<float>(), (long long)out.numel(), coef.data_ptr<float>(), (int)n, out.data_ptr<float>(),
                     (long long)out.numel(), stream()), "stack_mix");
}

int64_t router_max_outputs() { return r32_router_max_outputs(); }

// z fp32 [T, NE] router logits, corr fp32 [NE]; the first E outputs are real experts.  Returns
// (ids [T,k] i32, w [T,k] f32, row_off [E+1] i32, src [T*k] i32, row_expert [T*k] i32, inv [T*k] i32).
// bias fp32 [NE] is added to the logits; renorm: the chosen weights are divided by their sum (= softmax over the chosen).
std::vector<Tensor> router(Tensor z, c10::optional<Tensor> corr, int64_t E, int64_t k, c10::optional<Tensor> bias,
                           bool renorm) {
  want(z, torch::kFloat32, "router z");
  if (corr.has_value()) want(*corr, torch::kFloat32, "router correction");
  if (bias.has_value()) want(*bias, torch::kFloat32, "router bias");
  TORCH_CHECK(z.dim() == 2 && (!corr.has_value() || corr->numel() == z.size(1)) &&
                  (!bias.has_value() || bias->numel() == z.size(1)) && E >= 0 && E <= z.size(1) && k >= 1 && k <= z.size(1) &&
                  z.size(1) <= r32_router_max_outputs(), "router: shapes disagree");
  const int T = (int)z.size(0), NE = (int)z.size(1);
  auto oi = z.options().dtype(torch::kInt32);
  Tensor ids = torch::empty({T, k}, oi), w = torch::empty({T, k}, z.options()), rank = torch::empty({T, k}, oi);
  const int64_t Ec = std::max<int64_t>(E, 1);
  Tensor zeroed = torch::zeros({Ec + 2 * (int64_t)T * k}, oi);  // counts | src | row_expert: one fill
  Tensor counts = zeroed.narrow(0, 0, Ec), src = zeroed.narrow(0, Ec, T * k), row_expert = zeroed.narrow(0, Ec + T * k, T * k);
  Tensor row_off = torch::empty({E + 1}, oi), inv = torch::empty({T * k}, oi);
  done(r32_router(z.data_ptr<float>(), corr.has_value() ? corr->data_ptr<float>() : nullptr,
                  bias.has_value() ? bias->data_ptr<float>() : nullptr, renorm ? 1 : 0, T, NE, (int)E, (int)k, ids.data_ptr<int>(), w.data_ptr<float>(),
                  counts.data_ptr<int>(), rank.data_ptr<int>(), row_off.data_ptr<int>(), src.data_ptr<int>(),
                  row_expert.data_ptr<int>(), inv.data_ptr<int>(), stream()), "router");
  if (T == 0) row_off.zero_();
  return {ids, w, row_off, src, row_expert, inv};
}

// h [T, d]; w_gu [E, 2 ff, d] (gate rows, then up rows), w_down [E, d, ff]; returns Y fp32 [len(src), d] (rows beyond
// row_off[E] are not written)
Tensor expert_rows(Tensor h, Tensor src, Tensor row_expert, Tensor row_off, Tensor w_gu, Tensor w_down) {
  const int f = act_f32(h, "expert_rows h");
  const int ldh = row_stride(h, "expert_rows h");
  want(src, torch::kInt32, "expert_rows src");
  want(row_expert, torch::kInt32, "expert_rows row_expert");
  want(row_off, torch::kInt32, "expert_rows row_off");
  const int d = (int)h.size(1);
  TORCH_CHECK(w_gu.is_cuda() && w_down.is_cuda() && w_gu.is_contiguous() && w_down.is_contiguous() && w_gu.dim() == 3 &&
                  w_down.dim() == 3 && w_gu.scalar_type() == h.scalar_type() && w_down.scalar_type() == h.scalar_type() &&
                  w_gu.size(2) == d && w_down.size(1) == d && w_gu.size(1) == 2 * w_down.size(2) && w_gu.size(0) == w_down.size(0) &&
                  row_off.numel() == w_gu.size(0) + 1 && row_expert.numel() == src.numel(), "expert_rows: shapes or dtypes disagree");
  Tensor Y = torch::empty({src.numel(), d}, h.options().dtype(torch::kFloat32));
  done(r32_expert_rows(h.data_ptr(), ldh, src.data_ptr<int>(), row_expert.data_ptr<int>(), row_off.data_ptr<int>(),
                       (int)w_gu.size(0), w_gu.data_ptr(), w_down.data_ptr(), Y.data_ptr<float>(), (int)src.numel(), d,
                       (int)w_down.size(2), f, stream()), "expert_rows");
  return Y;
}

// out fp32 [T, d] = sum_j w[t][j] * (inv[t k + j] >= 0 ? Y[inv] : h[t])
// add: rows [T, d] of h's dtype added to every token's sum (a shared expert's result), or absent
Tensor moe_combine(Tensor Y, Tensor inv, Tensor w, Tensor h, c10::optional<Tensor> add) {
  const int f = act_f32(h, "moe_combine h"), fy = act_f32(Y, "moe_combine Y");
  const int ldh = row_stride(h, "moe_combine h");
  want(inv, torch::kInt32, "moe_combine inv");
  want(w, torch::kFloat32, "moe_combine w");
  const int T = (int)h.size(0), d = (int)h.size(1);
  TORCH_CHECK(w.dim() == 2 && w.size(0) == T && inv.numel() == w.numel() && Y.is_contiguous() && Y.dim() == 2 && Y.size(1) == d,
              "moe_combine: shapes disagree");
  Tensor out = torch::empty({T, d}, h.options().dtype(torch::kFloat32));
  const void* ap = nullptr;
  int lda = 0;
  if (add.has_value()) {
    TORCH_CHECK(add->is_cuda() && add->scalar_type() == h.scalar_type() && add->size(0) == T && add->size(1) == d,
                "moe_combine: add [T, d] of h's dtype");
    lda = row_stride(*add, "moe_combine add");
    ap = add->data_ptr();
  }
  done(r32_moe_combine(Y.data_ptr(), fy, inv.data_ptr<int>(), w.data_ptr<float>(), h.data_ptr(), ldh, T, (int)w.size(1),
                       out.data_ptr<float>(), d, ap, lda, f, stream()), "moe_combine");
  return out;
}

// Low-rank attention, cache side: proj rows [dq (Cq) | c (C) | rotated key part (R) | ...]; cq [T, Cq] receives the
// normalised query latent; the normalised c and the rotated part go to the K row (zeros up to nk), c again to the V row.
void latent_kv_write(Tensor proj, int64_t Cq, int64_t C, int64_t R, Tensor wq, Tensor wc, Tensor freq, double mult,
                     Tensor positions, Tensor slots, Tensor cq, Tensor k_cache, Tensor v_cache, double eps) {
  const int f = act_f32(proj, "latent_kv_write proj");
  const int ldp = row_stride(proj, "latent_kv_write proj"), ldq = row_stride(cq, "latent_kv_write cq");
  want(wq, torch::kFloat32, "latent_kv_write wq");
  want(wc, torch::kFloat32, "latent_kv_write wc");
  want(freq, torch::kFloat32, "latent_kv_write freq");
  want(positions, torch::kInt32, "latent_kv_write positions");
  want(slots, torch::kInt32, "latent_kv_write slots");
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "latent_kv_write");
  const int T = (int)proj.size(0);
  TORCH_CHECK(k_cache.scalar_type() == proj.scalar_type() && v_cache.scalar_type() == proj.scalar_type() &&
                  cq.scalar_type() == proj.scalar_type() && cq.is_cuda() && k_cache.is_cuda() && v_cache.is_cuda(),
              "latent_kv_write: one activation dtype");
  TORCH_CHECK(Cq >= 1 && C >= 1 && R >= 0 && R % 2 == 0 && proj.size(1) >= Cq + C + R && cq.size(0) == T && cq.size(1) == Cq &&
                  wq.numel() == Cq && wc.numel() == C && freq.numel() == R / 2 && positions.numel() == T && slots.numel() == T &&
                  nk >= C + R && nv >= C, "latent_kv_write: shapes disagree");
  done(r32_latent_kv_write(proj.data_ptr(), ldp, (int)Cq, (int)C, (int)R, wq.data_ptr<float>(), wc.data_ptr<float>(),
                           freq.data_ptr<float>(), (float)mult, positions.data_ptr<int>(), slots.data_ptr<int>(), cq.data_ptr(),
                           ldq, k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0),
                           (long long)v_cache.stride(0), BS, nk, nv, (float)eps, T, f, stream()), "latent_kv_write");
}

// q [T, H (D + R)] up-projected query rows; qn fp32 [H, T, C] their unrotated parts moved into the latent's space;
// out fp32 [T, H, Dk] = [qn scale | rot(q_rot) scale | 0]
// qn absent: the unrotated part is the rows' own (q[:, h, :D] * scale), out [T, H, Dk >= D + R]
void latent_q_rows(Tensor q, int64_t D, int64_t R, c10::optional<Tensor> qn_, Tensor freq, double mult, double scale,
                   Tensor positions, Tensor out, int64_t H) {
  const int f = act_f32(q, "latent_q_rows q");
  const int ldq = row_stride(q, "latent_q_rows q");
  if (!qn_.has_value()) {
    want(freq, torch::kFloat32, "latent_q_rows freq");
    want(positions, torch::kInt32, "latent_q_rows positions");
    want(out, torch::kFloat32, "latent_q_rows out");
    const int T = (int)q.size(0);
    TORCH_CHECK(out.dim() == 3 && out.size(0) == T && out.size(1) == H && q.size(1) == H * (D + R) && R % 2 == 0 &&
                    freq.numel() == R / 2 && positions.numel() == T && out.size(2) >= D + R, "latent_q_rows: shapes disagree");
    done(r32_latent_q_rows(q.data_ptr(), ldq, (int)D, (int)R, nullptr, (int)D, freq.data_ptr<float>(), (float)mult, (float)scale,
                           positions.data_ptr<int>(), out.data_ptr<float>(), (int)H, (int)out.size(2), T, f, stream()),
         "latent_q_rows");
    return;
  }
  Tensor qn = *qn_;
  want(qn, torch::kFloat32, "latent_q_rows qn");
  want(freq, torch::kFloat32, "latent_q_rows freq");
  want(positions, torch::kInt32, "latent_q_rows positions");
  want(out, torch::kFloat32, "latent_q_rows out");
  const int T = (int)q.size(0);
  TORCH_CHECK(qn.dim() == 3 && qn.size(0) == H && qn.size(1) == T && out.dim() == 3 && out.size(0) == T && out.size(1) == H &&
                  q.size(1) == H * (D + R) && R % 2 == 0 && freq.numel() == R / 2 && positions.numel() == T &&
                  out.size(2) >= qn.size(2) + R, "latent_q_rows: shapes disagree");
  done(r32_latent_q_rows(q.data_ptr(), ldq, (int)D, (int)R, qn.data_ptr<float>(), (int)qn.size(2), freq.data_ptr<float>(),
                         (float)mult, (float)scale, positions.data_ptr<int>(), out.data_ptr<float>(), (int)H, (int)out.size(2), T,
                         f, stream()), "latent_q_rows");
}

// Keys and values up-projected from cached latents into pages of their own: kv rows [N, H D + H Dv] (keys of all heads,
// then values), lat rows [N, >= rot_off + R] (the cached rows: the rotated key part at rot_off), slots int64 [N]; per
// token and head the key row [kv key (D) | rotated part (R) | zeros] of dk entries, the value row [value | zeros] of dv.
void latent_expand_write(Tensor kv, Tensor lat, int64_t rot_off, int64_t R, Tensor slots, Tensor k_cache, Tensor v_cache,
                         int64_t H, int64_t D, int64_t Dv) {
  const int f = act_f32(kv, "latent_expand_write kv");
  const int ldk = row_stride(kv, "latent_expand_write kv"), ldl = row_stride(lat, "latent_expand_write lat");
  want(slots, torch::kInt64, "latent_expand_write slots");
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "latent_expand_write");
  const int N = (int)kv.size(0);
  TORCH_CHECK(lat.is_cuda() && lat.scalar_type() == kv.scalar_type() && k_cache.scalar_type() == kv.scalar_type() &&
                  v_cache.scalar_type() == kv.scalar_type(), "latent_expand_write: one dtype");
  TORCH_CHECK(H > 0 && nk % H == 0 && nv % H == 0 && kv.size(1) == H * (D + Dv) && lat.size(0) == N && lat.size(1) >= rot_off + R &&
                  slots.numel() == N && nk / H >= D + R && nv / H >= Dv, "latent_expand_write: shapes disagree");
  done(r32_latent_expand_write(kv.data_ptr(), ldk, lat.data_ptr(), ldl, (int)rot_off, (const long long*)slots.data_ptr<int64_t>(),
                               k_cache.data_ptr(), v_cache.data_ptr(), (long long)k_cache.stride(0), (long long)v_cache.stride(0),
                               BS, N, (int)H, (int)D, (int)R, (int)Dv, (int)(nk / H), (int)(nv / H), f, stream()),
       "latent_expand_write");
}

int64_t retention_max_dim() { return r32_retention_max_dim(); }

// proj rows with q at column 0 and k at k_off (H heads of D each); v rows [T, H Dv] (a column slice is fine); state fp32
// [slots, H, D, Dv]; out fp32 [T, H Dv]
void retention(Tensor proj, int64_t k_off, Tensor v, Tensor freq, double mult, int64_t rd, Tensor decay, Tensor state, Tensor cu,
               Tensor item_slot, Tensor positions, Tensor out, int64_t H) {
  const int f = act_f32(proj, "retention proj");
  const int ldp = row_stride(proj, "retention proj"), ldv = row_stride(v, "retention v"), ldo = row_stride(out, "retention out");
  want(freq, torch::kFloat32, "retention freq");
  want(decay, torch::kFloat32, "retention decay");
  want(cu, torch::kInt32, "retention cu");
  want(item_slot, torch::kInt32, "retention item_slot");
  want(positions, torch::kInt32, "retention positions");
  want_dev(state, torch::kFloat32, "retention state");
  want_dev(out, torch::kFloat32, "retention out");
  TORCH_CHECK(v.is_cuda() && v.scalar_type() == proj.scalar_type(), "retention: v of proj's dtype");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.stride(3) == 1 && state.stride(2) == state.size(3) &&
                  state.stride(1) == state.size(2) * state.size(3), "retention: state [slots, H, D, Dv]");
  const int D = (int)state.size(2), Dv = (int)state.size(3), T = (int)proj.size(0);
  TORCH_CHECK(k_off >= H * D && proj.size(1) >= k_off + H * D && v.size(0) == T && v.size(1) == H * Dv && out.size(0) == T &&
                  out.size(1) == H * Dv && rd >= 0 && rd % 2 == 0 && rd <= D && freq.numel() == rd / 2 && decay.numel() == H &&
                  positions.numel() == T && cu.numel() == item_slot.numel() + 1 && D <= r32_retention_max_dim(),
              "retention: shapes disagree");
  Tensor qk = torch::empty({T, 2 * H * D}, out.options());
  done(r32_retention_prep(proj.data_ptr(), ldp, (int)k_off, freq.data_ptr<float>(), (float)mult, positions.data_ptr<int>(),
                          qk.data_ptr<float>(), T, (int)H, D, (int)rd, 1.0f / std::sqrt((float)D), f, stream()),
       "retention_prep");
  done(r32_retention(qk.data_ptr<float>(), v.data_ptr(), ldv, decay.data_ptr<float>(), state.data_ptr<float>(),
                     (long long)state.stride(0), cu.data_ptr<int>(), item_slot.data_ptr<int>(), positions.data_ptr<int>(),
                     out.data_ptr<float>(), ldo, (int)item_slot.numel(), (int)H, D, Dv, f, stream()), "retention");
}

// in rows [gate (n) | up (n)], out rows of n; mode 0 silu(g) u, 1 the clamped unit g' sigmoid(alpha g') (u' + 1)
void glu(Tensor in, Tensor out, int64_t mode, double alpha, double limit) {
  const int f = act_f32(in, "glu in");
  const int ldi = row_stride(in, "glu in"), ldo = row_stride(out, "glu out");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == in.scalar_type() && in.size(0) == out.size(0) && in.size(1) == 2 * out.size(1) &&
                  (mode == 0 || mode == 1), "glu: shapes or dtypes disagree");
  done(r32_glu(in.data_ptr(), ldi, out.data_ptr(), ldo, (int)in.size(0), (int)out.size(1), (int)mode, (float)alpha, (float)limit,
               f, stream()), "glu");
}

// out = z / 2 (1 + erf(z / sqrt 2)) over row-dense views of one dtype
void gelu(Tensor in, Tensor out) {
  const int f = act_f32(in, "gelu in");
  const int ldi = row_stride(in, "gelu in"), ldo = row_stride(out, "gelu out");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == in.scalar_type() && out.size(0) == in.size(0) && out.size(1) == in.size(1),
              "gelu: shapes or dtypes disagree");
  done(r32_gelu(in.data_ptr(), ldi, out.data_ptr(), ldo, (int)in.size(0), (int)in.size(1), f, stream()), "gelu");
}

const float* opt_f32(const c10::optional<Tensor>& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  want(*t, torch::kFloat32, name);
  TORCH_CHECK(t->numel() == n, name, ": wrong size");
  return t->data_ptr<float>();
}

// src rows [q (H D) | k (G D) | v (G Dv)] (bf16 or fp32); wq / wk fp32 [D] per-head norm weights or absent; freq fp32
// [rd / 2] (absent when rd == 0), vfreq fp32 [Dv / 2] or absent (values not rotated); q_out fp32 [T, H D]; caches: one
// layer's views of the paged pool.
void rot_kv_write(Tensor src, c10::optional<Tensor> wq, c10::optional<Tensor> wk, c10::optional<Tensor> freq, double mult,
                  int64_t rd, c10::optional<Tensor> vfreq, Tensor positions, Tensor slots, Tensor q_out, Tensor k_cache,
                  Tensor v_cache, int64_t H, int64_t G, double eps, double scale) {
  const int fi = act_f32(src, "rot_kv_write src"), fc = act_f32(k_cache, "rot_kv_write k_cache");
  const int lds = row_stride(src, "rot_kv_write src");
  const int T = (int)src.size(0);
  want(positions, torch::kInt32, "rot_kv_write positions");
  want(slots, torch::kInt32, "rot_kv_write slots");
  want(q_out, torch::kFloat32, "rot_kv_write q_out");
  TORCH_CHECK(v_cache.is_cuda() && v_cache.scalar_type() == k_cache.scalar_type() && (fi || !fc),
              "rot_kv_write: caches of one dtype, bf16 rows only into a bf16 cache");
  int NB, BS, nk, nv;
  cache_layout(k_cache, v_cache, NB, BS, nk, nv, "rot_kv_write");
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && nk % G == 0 && nv % G == 0, "rot_kv_write: head counts");
  const int D = nk / (int)G, Dv = nv / (int)G;
  TORCH_CHECK(src.size(1) == H * D + nk + nv && positions.numel() == T && slots.numel() == T &&
                  q_out.numel() == (int64_t)T * H * D && rd >= 0 && rd <= D && rd % 2 == 0 && (rd == 0 || freq.has_value()) &&
                  (!vfreq.has_value() || Dv % 2 == 0), "rot_kv_write: shapes disagree");
  done(r32_rot_kv_write(src.data_ptr(), lds, opt_f32(wq, D, "rot_kv_write wq"), opt_f32(wk, D, "rot_kv_write wk"),
                        opt_f32(freq, rd / 2, "rot_kv_write freq"), (float)mult, (int)rd, opt_f32(vfreq, Dv / 2, "rot_kv_write vfreq"),
                        positions.data_ptr<int>(), slots.data_ptr<int>(), q_out.data_ptr<float>(), k_cache.data_ptr(),
                        v_cache.data_ptr(), (long long)k_cache.stride(0), (long long)v_cache.stride(0), BS, T, (int)H, (int)G, D,
                        Dv, (float)eps, (float)scale, fi | (fc << 1), stream()), "rot_kv_write");
}

// o, out [T, H Dv] row-dense views of one dtype (not the same memory); g [T, >= H] gate logits or absent
void head_gate_unrotate(Tensor o, c10::optional<Tensor> g, c10::optional<Tensor> vfreq, Tensor positions, Tensor out,
                        int64_t H, double scale) {
  const int f = act_f32(o, "head_gate_unrotate o");
  const int ldi = row_stride(o, "head_gate_unrotate o"), ldo = row_stride(out, "head_gate_unrotate out");
  want(positions, torch::kInt32, "head_gate_unrotate positions");
  const int T = (int)o.size(0);
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == o.scalar_type() && out.size(0) == T && out.size(1) == o.size(1) && H > 0 &&
                  o.size(1) % H == 0 && positions.numel() == T && out.data_ptr() != o.data_ptr(), "head_gate_unrotate: shapes");
  const int Dv = (int)(o.size(1) / H);
  const void* gp = nullptr;
  int ldg = 0;
  if (g.has_value()) {
    TORCH_CHECK(g->is_cuda() && g->scalar_type() == o.scalar_type() && g->size(0) == T && g->size(1) == H, "head_gate_unrotate: g");
    ldg = row_stride(*g, "head_gate_unrotate g");
    gp = g->data_ptr();
  }
  done(r32_head_gate_unrotate(o.data_ptr(), ldi, gp, ldg, opt_f32(vfreq, Dv / 2, "head_gate_unrotate vfreq"),
                              positions.data_ptr<int>(), out.data_ptr(), ldo, T, (int)H, Dv, (float)scale, f, stream()),
       "head_gate_unrotate");
}

// x fp32 [T, d] += y (absent: x stays); out = x / rms(x) * w (bf16 or fp32 rows)
void add_rmsnorm(Tensor x, c10::optional<Tensor> y, Tensor w, Tensor out, double eps) {
  want(x, torch::kFloat32, "add_rmsnorm x");
  want(w, torch::kFloat32, "add_rmsnorm w");
  const int fo = act_f32(out, "add_rmsnorm out");
  const int ldo = row_stride(out, "add_rmsnorm out");
  TORCH_CHECK(x.dim() == 2 && out.size(0) == x.size(0) && out.size(1) == x.size(1) && w.numel() == x.size(1), "add_rmsnorm: shapes");
  const void* yp = nullptr;
  int ldy = 0, fy = 0;
  if (y.has_value()) {
    fy = act_f32(*y, "add_rmsnorm y");
    ldy = row_stride(*y, "add_rmsnorm y");
    TORCH_CHECK(y->size(0) == x.size(0) && y->size(1) == x.size(1), "add_rmsnorm: y");
    yp = y->data_ptr();
  }
  done(r32_add_rmsnorm(x.data_ptr<float>(), yp, ldy, w.data_ptr<float>(), out.data_ptr(), ldo, (int)x.size(0), (int)x.size(1),
                       (float)eps, fy | (fo << 1), stream()), "add_rmsnorm");
}

int64_t chan_rule_max_dim() { return r32_chan_rule_max_dim(); }

// src [T, 2 G D + H Dv] rows [q | k | v] (bf16 or fp32); qkv fp32 of the same shape (src itself when that is fp32);
// z [T, H D] decay logits, zb fp32 [H D] or absent; A_log fp32 [H] (delta-rule decays) or absent (sigmoid^(1/tau));
// b [T, >= H] beta logits or absent; state fp32 [slots, H, D, Dv] view; out fp32 [T, H Dv].
void chan_rule(Tensor src, Tensor qkv, Tensor z, c10::optional<Tensor> zb, c10::optional<Tensor> A_log, double inv_tau,
               c10::optional<Tensor> b, Tensor state, Tensor cu, Tensor item_slot, Tensor positions, Tensor out, int64_t H,
               int64_t G, bool unit, bool delta) {
  const int fs = act_f32(src, "chan_rule src"), fz = act_f32(z, "chan_rule z");
  const int lds = row_stride(src, "chan_rule src"), ldz = row_stride(z, "chan_rule z");
  want_dev(qkv, torch::kFloat32, "chan_rule qkv");
  const int ldq = row_stride(qkv, "chan_rule qkv");
  want_dev(state, torch::kFloat32, "chan_rule state");
  want(cu, torch::kInt32, "chan_rule cu");
  want(item_slot, torch::kInt32, "chan_rule item_slot");
  want(positions, torch::kInt32, "chan_rule positions");
  want_dev(out, torch::kFloat32, "chan_rule out");
  const int ldo = row_stride(out, "chan_rule out");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.stride(3) == 1 && state.stride(2) == state.size(3) &&
                  state.stride(1) == state.size(2) * state.size(3), "chan_rule: state [slots, H, D, Dv]");
  const int D = (int)state.size(2), Dv = (int)state.size(3), T = (int)src.size(0);
  TORCH_CHECK(G > 0 && H % G == 0 && src.size(1) == 2 * G * D + H * Dv && qkv.size(0) == T && qkv.size(1) == src.size(1) &&
                  out.size(0) == T && out.size(1) == H * Dv && z.size(0) == T && z.size(1) == H * D && positions.numel() == T &&
                  cu.numel() == item_slot.numel() + 1 && D <= r32_chan_rule_max_dim() &&
                  (fs || src.data_ptr() != qkv.data_ptr()), "chan_rule: shapes disagree");
  const void* bp = nullptr;
  int ldb = 0, fb = 0;
  if (b.has_value()) {
    fb = act_f32(*b, "chan_rule b");
    ldb = row_stride(*b, "chan_rule b");
    TORCH_CHECK(b->size(0) == T && b->size(1) == H, "chan_rule: b [T, H]");
    bp = b->data_ptr();
  }
  Tensor dec = torch::empty({T, H * D}, qkv.options().dtype(torch::kFloat32));
  Tensor bq = torch::empty({T, H + G}, dec.options());
  done(r32_chan_rule(src.data_ptr(), lds, fs, qkv.data_ptr<float>(), ldq, z.data_ptr(), ldz, fz,
                     opt_f32(zb, H * D, "chan_rule zb"), opt_f32(A_log, H, "chan_rule A_log"), (float)inv_tau, bp, ldb, fb,
                     dec.data_ptr<float>(), bq.data_ptr<float>(), state.data_ptr<float>(), (long long)state.stride(0),
                     cu.data_ptr<int>(), item_slot.data_ptr<int>(), positions.data_ptr<int>(), out.data_ptr<float>(), ldo, T,
                     (int)item_slot.numel(), (int)H, (int)G, D, Dv, unit ? 1 : 0, delta ? 1 : 0, stream()), "chan_rule");
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
  m.def("window_attn_decode_ok", &window_attn_decode_ok);
  m.def("window_attn_decode", &window_attn_decode);
  m.def("conv_hist", &conv_hist);
  m.def("conv_hist_update", &conv_hist_update);
  m.def("delta_rule", &delta_rule);
  m.def("delta_rule_max_dim", &delta_rule_max_dim);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("embed_rows", &embed_rows);
  m.def("head_norm_kv_write", &head_norm_kv_write);
  m.def("gate_mul", &gate_mul);
  m.def("gated_norm_residual", &gated_norm_residual);
  m.def("rmsnorm_rows", &rmsnorm_rows);
  m.def("gelu_mul_rows", &gelu_mul_rows);
  m.def("stack_mix", &stack_mix);
  m.def("router", &router);
  m.def("router_max_outputs", &router_max_outputs);
  m.def("expert_rows", &expert_rows);
  m.def("moe_combine", &moe_combine);
  m.def("latent_kv_write", &latent_kv_write);
  m.def("latent_q_rows", &latent_q_rows);
  m.def("latent_expand_write", &latent_expand_write);
  m.def("retention", &retention);
  m.def("retention_max_dim", &retention_max_dim);
  m.def("glu", &glu);
  m.def("gelu", &gelu);
  m.def("rot_kv_write", &rot_kv_write);
  m.def("head_gate_unrotate", &head_gate_unrotate);
  m.def("add_rmsnorm", &add_rmsnorm);
  m.def("chan_rule", &chan_rule);
  m.def("chan_rule_max_dim", &chan_rule_max_dim);
}

// Layer plumbing of fp32-residual designs with gated, post-normalised sublayers (gfx950, wave64).
//
//   embed_rows           x[t] = table[token[t]] * scale as fp32
//   head_norm_kv_write   from fused projection rows: q and k divided by their root mean square PER HEAD (no weight);
//                        q times scale * (1 + coef ln(floor((p + 1) / every) + 1)) into an fp32 buffer; normalised k
//                        into the paged K cache; the values (a projection of their own, or the keys as projected,
//                        before the norm) into the 4-token interleaved paged V cache
//   gate_mul             a *= sigmoid(g) (or silu(g)), column slices of row-dense buffers
//   gated_norm_residual  x += z / rms(z) * w with z = y * sigmoid(r) (or z = y): the sublayer's gated, normalised
//                        result added to the fp32 residual stream (optionally also a bf16 copy of the new x)
//   rmsnorm_rows         out[n] = x[rows[n]] / rms * w (fp32 rows in, activation dtype out)
//   gelu_mul_rows        out[t][c] = gelu_tanh(z[t][c]) * table[token[t]][off + c]
//   stack_mix            out = sum_j coef[j] * X[j] over a stack of fp32 streams
#include "elem.h"

namespace lwc {
namespace {

template <typename AT>
__global__ void embed_rows_kernel(const AT* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ out,
                                  int d, int vocab, float scale) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const AT* row = table + (size_t)tok * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[(size_t)t * d + i] = Elem<AT>::ld(row + i) * scale;
}

// proj row t: q at column 0 (H*D), k at k_off (G*D), values at v_off (G*Dv; v_off == k_off: the keys as projected).
template <typename AT>
__global__ void head_norm_kv_write_kernel(const AT* __restrict__ proj, int ldp, int k_off, int v_off,
                                          const int* __restrict__ positions, const int* __restrict__ slots,
                                          float* __restrict__ q_out, AT* __restrict__ k_cache, AT* __restrict__ v_cache,
                                          long long kb_stride, long long vb_stride, int block_size, int H, int G, int D,
                                          int Dv, float eps, float scale, float coef, int every) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const AT* pr = proj + (size_t)t * ldp;
  const int p = positions[t];
  const float qmul = scale * (1.0f + (every > 0 ? coef * logf((float)((p + 1) / every) + 1.0f) : 0.f));
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  const int nk = G * D, nv = G * Dv;
  for (int h = wv; h < H + G; h += nw) {
    const bool isq = h < H;
    const AT* src = isq ? pr + h * D : pr + k_off + (h - H) * D;
    float s = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = Elem<AT>::ld(src + i);
      s += v * v;
    }
    const float rstd = 1.0f / sqrtf(wave_sum(s) / (float)D + eps);
    if (isq) {
      float* qo = q_out + (size_t)t * H * D + h * D;
      for (int i = lane; i < D; i += 64) qo[i] = Elem<AT>::ld(src + i) * rstd * qmul;
    } else if (write) {
      const int g = h - H;
      AT* kc = k_cache + blk * kb_stride + off * nk + g * D;
      for (int i = lane; i < D; i += 64) Elem<AT>::st(kc + i, Elem<AT>::ld(src + i) * rstd);
      // V is 4-token interleaved: [block][offset / 4][column][offset % 4]
      AT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3) + 4LL * g * Dv;
      const AT* vs = pr + v_off + g * Dv;
      for (int i = lane; i < Dv; i += 64) vc[4 * i] = vs[i];
    }
  }
}

// D / 4 (and Dv / 4) a power of two <= 64, every base a multiple of four elements: LPH = D / 4 lanes per head and
// 64 / LPH heads per wave at once; 8- / 16-byte loads and stores except the interleaved value stores.
template <typename AT>
__global__ void head_norm_kv_write_sub_kernel(const AT* __restrict__ proj, int ldp, int k_off, int v_off,
                                              const int* __restrict__ positions, const int* __restrict__ slots,
                                              float* __restrict__ q_out, AT* __restrict__ k_cache, AT* __restrict__ v_cache,
                                              long long kb_stride, long long vb_stride, int block_size, int H, int G, int D,
                                              float eps, float scale, float coef, int every, int LPH) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int hpw = 64 / LPH, sub = lane / LPH, i = (lane - sub * LPH) * 4;
  const AT* pr = proj + (size_t)t * ldp;
  const int p = positions[t];
  const float qmul = scale * (1.0f + (every > 0 ? coef * logf((float)((p + 1) / every) + 1.0f) : 0.f));
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  const int nk = G * D;
  for (int h0 = wv * hpw; h0 < H + G; h0 += nw * hpw) {
    const int h = h0 + sub;
    const bool ok = h < H + G, isq = h < H;
    const AT* src = !ok ? pr : (isq ? pr + h * D : pr + k_off + (h - H) * D);
    const float4v v = Vec4<AT>::ld(src + i);
    float s = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    for (int m = LPH >> 1; m > 0; m >>= 1) s += __shfl_xor(s, m, 64);
    const float rstd = 1.0f / sqrtf(s / (float)D + eps);
    if (!ok) continue;
    if (isq) {
      Vec4<float>::st(q_out + (size_t)t * H * D + h * D + i, v * (rstd * qmul));
    } else if (write) {
      const int g = h - H;
      Vec4<AT>::st(k_cache + blk * kb_stride + off * nk + g * D + i, v * rstd);
      // V is 4-token interleaved: [block][offset / 4][column][offset % 4]; here the values are D wide like the keys
      AT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nk) + (off & 3) + 4LL * (g * D + i);
      const AT* vs = pr + v_off + g * D + i;
#pragma unroll
      for (int e = 0; e < 4; ++e) vc[4 * e] = vs[e];
    }
  }
}

template <typename AT, int MODE>
__global__ void gate_mul_kernel(AT* __restrict__ a, int lda, const AT* __restrict__ g, int ldg, int n, long long total) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    const long long r = e / n;
    const int c = (int)(e - r * n);
    const float z = Elem<AT>::ld(g + r * ldg + c);
    AT* p = a + r * lda + c;
    Elem<AT>::st(p, Elem<AT>::ld(p) * (MODE == 0 ? sigmoid_f(z) : silu_f(z)));
  }
}

template <typename AT, int MODE>
__global__ void gate_mul_vec_kernel(AT* __restrict__ a, int lda, const AT* __restrict__ g, int ldg, int n4, long long total4) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total4; e += (long long)gridDim.x * blockDim.x) {
    const long long r = e / n4;
    const int c = (int)(e - r * n4) * 4;
    const float4v z = Vec4<AT>::ld(g + r * ldg + c);
    AT* p = a + r * lda + c;
    const float4v m = MODE == 0 ? float4v{sigmoid_f(z[0]), sigmoid_f(z[1]), sigmoid_f(z[2]), sigmoid_f(z[3])}
                                : float4v{silu_f(z[0]), silu_f(z[1]), silu_f(z[2]), silu_f(z[3])};
    Vec4<AT>::st(p, Vec4<AT>::ld(p) * m);
  }
}

template <typename YT, typename GT>
__global__ void gated_norm_residual_kernel(float* __restrict__ x, const YT* __restrict__ y, int ldy,
                                           const GT* __restrict__ r, int ldr, const float* __restrict__ w,
                                           bf16_t* __restrict__ x_cast, const float* __restrict__ w_next, int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const YT* yr = y + (size_t)t * ldy;
  const GT* rr = r ? r + (size_t)t * ldr : nullptr;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float z = Elem<YT>::ld(yr + i);
    if (rr) z *= sigmoid_f(Elem<GT>::ld(rr + i));
    s += z * z;
  }
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
  float* xr = x + (size_t)t * d;
  float s2 = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float z = Elem<YT>::ld(yr + i);
    if (rr) z *= sigmoid_f(Elem<GT>::ld(rr + i));
    const float v = xr[i] + z * rstd * w[i];
    xr[i] = v;
    s2 += v * v;
    if (x_cast && !w_next) x_cast[(size_t)t * d + i] = f2bf(v);
  }
  if (x_cast && w_next) {  // the next sublayer's input norm of the new x (each thread re-reads what it wrote)
    const float rstd2 = 1.0f / sqrtf(block_sum(s2, scratch) / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) x_cast[(size_t)t * d + i] = f2bf(xr[i] * rstd2 * w_next[i]);
  }
}

// Rows of d <= 4 * 256 * NCH elements, every base a multiple of four elements: z stays in registers between the sum
// of squares and the update; 16-byte accesses of x.
template <typename YT, typename GT, int NCH>
__global__ void __launch_bounds__(256) gated_norm_residual_vec_kernel(float* __restrict__ x, const YT* __restrict__ y, int ldy,
                                                                       const GT* __restrict__ r, int ldr,
                                                                       const float* __restrict__ w,
                                                                       bf16_t* __restrict__ x_cast,
                                                                       const float* __restrict__ w_next, int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const YT* yr = y + (size_t)t * ldy;
  const GT* rr = r ? r + (size_t)t * ldr : nullptr;
  float4v z[NCH];
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    z[u] = float4v{0.f, 0.f, 0.f, 0.f};
    if (i < d) {
      z[u] = Vec4<YT>::ld(yr + i);
      if (rr) {
        const float4v g = Vec4<GT>::ld(rr + i);
        z[u] *= float4v{sigmoid_f(g[0]), sigmoid_f(g[1]), sigmoid_f(g[2]), sigmoid_f(g[3])};
      }
      s += z[u][0] * z[u][0] + z[u][1] * z[u][1] + z[u][2] * z[u][2] + z[u][3] * z[u][3];
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
  float* xr = x + (size_t)t * d;
  float s2 = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    if (i < d) {
      const float4v v = Vec4<float>::ld(xr + i) + z[u] * rstd * Vec4<float>::ld(w + i);
      Vec4<float>::st(xr + i, v);
      if (x_cast && !w_next) Vec4<bf16_t>::st(x_cast + (size_t)t * d + i, v);
      z[u] = v;
      s2 += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
  }
  if (x_cast && w_next) {  // the next sublayer's input norm of the new x, from registers
    const float rstd2 = 1.0f / sqrtf(block_sum(s2, scratch) / (float)d + eps);
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
      const int i = (threadIdx.x + 256 * u) * 4;
      if (i < d) Vec4<bf16_t>::st(x_cast + (size_t)t * d + i, z[u] * rstd2 * Vec4<float>::ld(w_next + i));
    }
  }
}

template <typename AT>
__global__ void rmsnorm_rows_kernel(const float* __restrict__ x, const long long* __restrict__ rows,
                                    const float* __restrict__ w, AT* __restrict__ out, int d, float eps) {
  __shared__ float scratch[16];
  const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const float* xr = x + r * d;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) s += xr[i] * xr[i];
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) Elem<AT>::st(out + (size_t)blockIdx.x * d + i, xr[i] * rstd * w[i]);
}

// d <= 4 * 256 * NCH, a multiple of four, aligned bases: the row is read once and stays in registers
template <typename AT, int NCH>
__global__ void __launch_bounds__(256) rmsnorm_rows_vec_kernel(const float* __restrict__ x, const long long* __restrict__ rows,
                                                                const float* __restrict__ w, AT* __restrict__ out, int d,
                                                                float eps) {
  __shared__ float scratch[16];
  const size_t r = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  const float* xr = x + r * d;
  float4v v[NCH];
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    v[u] = float4v{0.f, 0.f, 0.f, 0.f};
    if (i < d) {
      v[u] = Vec4<float>::ld(xr + i);
      s += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    if (i < d) Vec4<AT>::st(out + (size_t)blockIdx.x * d + i, v[u] * rstd * Vec4<float>::ld(w + i));
  }
}

template <typename AT>
__global__ void gelu_mul_rows_kernel(const AT* __restrict__ z, int ldz, const AT* __restrict__ table, int ldt, int off,
                                     const int* __restrict__ tokens, int vocab, AT* __restrict__ out, int n, int T) {
  const long long total = (long long)T * n;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    const long long t = e / n;
    const int c = (int)(e - t * n);
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    Elem<AT>::st(out + t * n + c, gelu_tanh_f(Elem<AT>::ld(z + t * ldz + c)) * Elem<AT>::ld(table + (size_t)tok * ldt + off + c));
  }
}

__global__ void stack_mix_vec_kernel(const float* __restrict__ X, long long plane, const float* __restrict__ coef, int n,
                                     float* __restrict__ out, long long total4) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total4; e += (long long)gridDim.x * blockDim.x) {
    float4v s = float4v{0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < n; ++j) s += Vec4<float>::ld(X + j * plane + 4 * e) * coef[j];
    Vec4<float>::st(out + 4 * e, s);
  }
}

__global__ void stack_mix_kernel(const float* __restrict__ X, long long plane, const float* __restrict__ coef, int n,
                                 float* __restrict__ out, long long total) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    float s = 0.f;
    for (int j = 0; j < n; ++j) s += coef[j] * X[j * plane + e];
    out[e] = s;
  }
}

int blocks_for(long long total) { return (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536); }

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_embed_rows(const void* table, const int* tokens, float* out, int T, int d, int vocab, float scale,
                              int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (f32) embed_rows_kernel<float><<<T, 256, 0, s>>>((const float*)table, tokens, out, d, vocab, scale);
  else embed_rows_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)table, tokens, out, d, vocab, scale);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_head_norm_kv_write(const void* proj, int ldp, int k_off, int v_off, const int* positions,
                                      const int* slots, float* q_out, void* k_cache, void* v_cache, long long kb_stride,
                                      long long vb_stride, int block_size, int T, int H, int G, int D, int Dv, float eps,
                                      float scale, float coef, int every, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  const int lph = D / 4, ab = f32 ? 16 : 8;
  if (D == Dv && D % 4 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 && ldp % 4 == 0 && k_off % 4 == 0 && v_off % 4 == 0 &&
      kb_stride % 4 == 0 && aligned_to(proj, ab) && aligned_to(k_cache, ab) && aligned_to(q_out, 16)) {
    if (f32)
      head_norm_kv_write_sub_kernel<float><<<T, 256, 0, s>>>((const float*)proj, ldp, k_off, v_off, positions, slots, q_out,
                                                              (float*)k_cache, (float*)v_cache, kb_stride, vb_stride,
                                                              block_size, H, G, D, eps, scale, coef, every, lph);
    else
      head_norm_kv_write_sub_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)proj, ldp, k_off, v_off, positions, slots,
                                                               q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride,
                                                               vb_stride, block_size, H, G, D, eps, scale, coef, every, lph);
    LWC_CHECK_LAUNCH();
    return 0;
  }
  if (f32)
    head_norm_kv_write_kernel<float><<<T, 256, 0, s>>>((const float*)proj, ldp, k_off, v_off, positions, slots, q_out,
                                                        (float*)k_cache, (float*)v_cache, kb_stride, vb_stride, block_size, H,
                                                        G, D, Dv, eps, scale, coef, every);
  else
    head_norm_kv_write_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)proj, ldp, k_off, v_off, positions, slots, q_out,
                                                         (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride, vb_stride, block_size,
                                                         H, G, D, Dv, eps, scale, coef, every);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_gate_mul(void* a, int lda, const void* g, int ldg, int T, int n, int mode, int f32, hipStream_t s) {
  const long long total = (long long)T * n;
  if (total <= 0) return 0;
  if (n % 4 == 0 && lda % 4 == 0 && ldg % 4 == 0 && aligned_to(a, f32 ? 16 : 8) && aligned_to(g, f32 ? 16 : 8)) {
    const int nb4 = blocks_for(total / 4);
    if (f32) {
      if (mode == 0) gate_mul_vec_kernel<float, 0><<<nb4, 256, 0, s>>>((float*)a, lda, (const float*)g, ldg, n / 4, total / 4);
      else gate_mul_vec_kernel<float, 1><<<nb4, 256, 0, s>>>((float*)a, lda, (const float*)g, ldg, n / 4, total / 4);
    } else {
      if (mode == 0) gate_mul_vec_kernel<bf16_t, 0><<<nb4, 256, 0, s>>>((bf16_t*)a, lda, (const bf16_t*)g, ldg, n / 4, total / 4);
      else gate_mul_vec_kernel<bf16_t, 1><<<nb4, 256, 0, s>>>((bf16_t*)a, lda, (const bf16_t*)g, ldg, n / 4, total / 4);
    }
    LWC_CHECK_LAUNCH();
    return 0;
  }
  const int nb = blocks_for(total);
  if (f32) {
    if (mode == 0) gate_mul_kernel<float, 0><<<nb, 256, 0, s>>>((float*)a, lda, (const float*)g, ldg, n, total);
    else gate_mul_kernel<float, 1><<<nb, 256, 0, s>>>((float*)a, lda, (const float*)g, ldg, n, total);
  } else {
    if (mode == 0) gate_mul_kernel<bf16_t, 0><<<nb, 256, 0, s>>>((bf16_t*)a, lda, (const bf16_t*)g, ldg, n, total);
    else gate_mul_kernel<bf16_t, 1><<<nb, 256, 0, s>>>((bf16_t*)a, lda, (const bf16_t*)g, ldg, n, total);
  }
  LWC_CHECK_LAUNCH();
  return 0;
}

// y_f32 / r_f32: element types of the sublayer result and of the gate logits (r may be null: no gate)
extern "C" int r32_gated_norm_residual(float* x, const void* y, int ldy, const void* r, int ldr, const float* w,
                                       void* x_cast, const float* w_next, int T, int d, float eps, int y_f32, int r_f32,
                                       hipStream_t s) {
  if (T <= 0) return 0;
  const bool vec = d % 4 == 0 && d <= 8192 && ldy % 4 == 0 && ldr % 4 == 0 && aligned_to(x, 16) && aligned_to(w, 16) &&
                   aligned_to(w_next, 16) &&
                   aligned_to(y, y_f32 ? 16 : 8) && aligned_to(r, r_f32 ? 16 : 8) && aligned_to(x_cast, 8);
  if (vec) {
    const int nch = (d + 1023) / 1024;
#define LWC_GNR(YT, GT)                                                                                                  \
  if (nch <= 1)                                                                                                          \
    gated_norm_residual_vec_kernel<YT, GT, 1><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, (const GT*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps); \
  else if (nch <= 2)                                                                                                     \
    gated_norm_residual_vec_kernel<YT, GT, 2><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, (const GT*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps); \
  else if (nch <= 4)                                                                                                     \
    gated_norm_residual_vec_kernel<YT, GT, 4><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, (const GT*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps); \
  else                                                                                                                   \
    gated_norm_residual_vec_kernel<YT, GT, 8><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, (const GT*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps)
    if (y_f32 && (r_f32 || !r)) {
      LWC_GNR(float, float);
    } else if (y_f32) {
      LWC_GNR(float, bf16_t);
    } else if (!r_f32 || !r) {
      LWC_GNR(bf16_t, bf16_t);
    } else {
      return -1;
    }
#undef LWC_GNR
    LWC_CHECK_LAUNCH();
    return 0;
  }
  if (y_f32 && (r_f32 || !r))
    gated_norm_residual_kernel<float, float><<<T, 256, 0, s>>>(x, (const float*)y, ldy, (const float*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps);
  else if (y_f32)
    gated_norm_residual_kernel<float, bf16_t><<<T, 256, 0, s>>>(x, (const float*)y, ldy, (const bf16_t*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps);
  else if (!r_f32 || !r)
    gated_norm_residual_kernel<bf16_t, bf16_t><<<T, 256, 0, s>>>(x, (const bf16_t*)y, ldy, (const bf16_t*)r, ldr, w, (bf16_t*)x_cast, w_next, d, eps);
  else
    return -1;
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_rmsnorm_rows(const float* x, const long long* rows, const float* w, void* out, int n, int d, float eps,
                                int f32, hipStream_t s) {
  if (n <= 0) return 0;
  if (d % 4 == 0 && d <= 8192 && aligned_to(x, 16) && aligned_to(w, 16) && aligned_to(out, f32 ? 16 : 8)) {
    const int nch = (d + 1023) / 1024;
#define LWC_RMS(AT)                                                                                  \
  if (nch <= 1) rmsnorm_rows_vec_kernel<AT, 1><<<n, 256, 0, s>>>(x, rows, w, (AT*)out, d, eps);      \
  else if (nch <= 2) rmsnorm_rows_vec_kernel<AT, 2><<<n, 256, 0, s>>>(x, rows, w, (AT*)out, d, eps); \
  else if (nch <= 4) rmsnorm_rows_vec_kernel<AT, 4><<<n, 256, 0, s>>>(x, rows, w, (AT*)out, d, eps); \
  else rmsnorm_rows_vec_kernel<AT, 8><<<n, 256, 0, s>>>(x, rows, w, (AT*)out, d, eps)
    if (f32) {
      LWC_RMS(float);
    } else {
      LWC_RMS(bf16_t);
    }
#undef LWC_RMS
    LWC_CHECK_LAUNCH();
    return 0;
  }
  if (f32) rmsnorm_rows_kernel<float><<<n, 256, 0, s>>>(x, rows, w, (float*)out, d, eps);
  else rmsnorm_rows_kernel<bf16_t><<<n, 256, 0, s>>>(x, rows, w, (bf16_t*)out, d, eps);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_gelu_mul_rows(const void* z, int ldz, const void* table, int ldt, int off, const int* tokens, int vocab,
                                 void* out, int T, int n, int f32, hipStream_t s) {
  const long long total = (long long)T * n;
  if (total <= 0) return 0;
  const int nb = blocks_for(total);
  if (f32) gelu_mul_rows_kernel<float><<<nb, 256, 0, s>>>((const float*)z, ldz, (const float*)table, ldt, off, tokens, vocab, (float*)out, n, T);
  else gelu_mul_rows_kernel<bf16_t><<<nb, 256, 0, s>>>((const bf16_t*)z, ldz, (const bf16_t*)table, ldt, off, tokens, vocab, (bf16_t*)out, n, T);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_stack_mix(const float* X, long long plane, const float* coef, int n, float* out, long long total,
                             hipStream_t s) {
  if (total <= 0 || n <= 0) return 0;
  if (total % 4 == 0 && plane % 4 == 0 && aligned_to(X, 16) && aligned_to(out, 16))
    stack_mix_vec_kernel<<<blocks_for(total / 4), 256, 0, s>>>(X, plane, coef, n, out, total / 4);
  else
    stack_mix_kernel<<<blocks_for(total), 256, 0, s>>>(X, plane, coef, n, out, total);
  LWC_CHECK_LAUNCH();
  return 0;
}

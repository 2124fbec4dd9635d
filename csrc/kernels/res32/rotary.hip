// Rotations by position around the paged cache of a rotary attention layer (gfx950, wave64); arithmetic fp32.
//
//   rot_kv_write        from rows [q (H*D) | k (G*D) | v (G*Dv)]: q and k optionally RMS-normed per head (a weight of
//                       D entries shared by the heads), then their first `rd` entries rotated: entry i < rd/2 is paired
//                       with entry i + rd/2, the pair (u, v) at position p becomes
//                       (u c - v s, v c + u s), c = mult cos(p f_i), s = mult sin(p f_i);
//                       q times `scale` -> fp32 [T, H*D]; k -> paged K cache; v, optionally rotated the same way over
//                       all Dv entries by its own frequencies (no multiplier) -> 4-token interleaved paged V cache
//   head_gate_unrotate  out[t, h, :] = rot(o[t, h, :], -p) * sigmoid(g[t, h]) * scale: an attention output over rotated
//                       values turned back by the query's position, one gate per head (rotation optional)
//   add_rmsnorm         x (fp32) += y;  out = x / rms(x) * w: the residual sum and the next sublayer's input norm
#include "elem.h"

namespace lwc {
namespace {

// one head: D entries at src (norm optional), rotated on the first rd, times mul; dst(i, value) stores entry i
template <typename IT, typename ST>
LWC_DEVICE void rotate_head(const IT* src, int D, const float* w, float eps, int rd, const float* freq, float mult, float pos,
                            float mul, int lane, ST store) {
  float rstd = 1.0f;
  if (w) {
    float s = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = Elem<IT>::ld(src + i);
      s += v * v;
    }
    rstd = 1.0f / sqrtf(wave_sum(s) / (float)D + eps);
  }
  const int half = rd >> 1;
  for (int i = lane; i < D; i += 64) {
    float x = Elem<IT>::ld(src + i) * (w ? rstd * w[i] : 1.0f);
    if (i < rd) {
      const bool first = i < half;
      const int m = first ? i : i - half, j = first ? i + half : i - half;
      const float xp = Elem<IT>::ld(src + j) * (w ? rstd * w[j] : 1.0f);
      float sn, cs;
      sincosf(pos * freq[m], &sn, &cs);
      sn *= mult, cs *= mult;
      x = first ? x * cs - xp * sn : x * cs + xp * sn;
    }
    store(i, x * mul);
  }
}

template <typename IT, typename CT>
__global__ void rot_kv_write_kernel(const IT* __restrict__ src, int lds, const float* __restrict__ wq,
                                    const float* __restrict__ wk, const float* __restrict__ freq, float mult, int rd,
                                    const float* __restrict__ vfreq, const int* __restrict__ positions,
                                    const int* __restrict__ slots, float* __restrict__ q_out, CT* __restrict__ k_cache,
                                    CT* __restrict__ v_cache, long long kb_stride, long long vb_stride, int block_size,
                                    int H, int G, int D, int Dv, float eps, float scale) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const IT* pr = src + (size_t)t * lds;
  const float pos = (float)positions[t];
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  for (int h = wv; h < H + 2 * G; h += nw) {
    if (h < H) {
      float* qo = q_out + (size_t)t * nq + (size_t)h * D;
      rotate_head<IT>(pr + (size_t)h * D, D, wq, eps, rd, freq, mult, pos, scale, lane, [&](int i, float v) { qo[i] = v; });
    } else if (!write) {
      continue;
    } else if (h < H + G) {
      const int g = h - H;
      CT* kc = k_cache + blk * kb_stride + off * nk + (size_t)g * D;
      rotate_head<IT>(pr + nq + (size_t)g * D, D, wk, eps, rd, freq, mult, pos, 1.0f, lane,
                      [&](int i, float v) { Elem<CT>::st(kc + i, v); });
    } else {
      const int g = h - H - G;
      // V is 4-token interleaved: [block][offset / 4][column][offset % 4]
      CT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3) + 4LL * g * Dv;
      rotate_head<IT>(pr + nq + nk + (size_t)g * Dv, Dv, nullptr, eps, vfreq ? Dv : 0, vfreq, 1.0f, pos, 1.0f, lane,
                      [&](int i, float v) { Elem<CT>::st(vc + 4 * i, v); });
    }
  }
}

template <typename AT>
__global__ void head_gate_unrotate_kernel(const AT* __restrict__ o, int ldi, const AT* __restrict__ g, int ldg,
                                          const float* __restrict__ vfreq, const int* __restrict__ positions,
                                          AT* __restrict__ out, int ldo, int H, int Dv, float scale) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float pos = -(float)positions[t];   // turned back: the angles' signs flip
  for (int h = wv; h < H; h += nw) {
    const float gate = scale * (g ? sigmoid_f(Elem<AT>::ld(g + (size_t)t * ldg + h)) : 1.0f);
    AT* dst = out + (size_t)t * ldo + (size_t)h * Dv;
    rotate_head<AT>(o + (size_t)t * ldi + (size_t)h * Dv, Dv, nullptr, 0.f, vfreq ? Dv : 0, vfreq, 1.0f, pos, gate, lane,
                    [&](int i, float v) { Elem<AT>::st(dst + i, v); });
  }
}

// cos / sin of one row's angles, shared by all heads: tab[m] = mult cos(pos f_m), tab[n + m] = mult sin(pos f_m)
LWC_DEVICE void angle_table(float* tab, const float* freq, int n, float mult, float pos) {
  for (int m = threadIdx.x; m < n; m += blockDim.x) {
    float sn, cs;
    sincosf(pos * freq[m], &sn, &cs);
    tab[m] = cs * mult;
    tab[n + m] = sn * mult;
  }
}

// four consecutive entries [i, i + 4) of a head at src, rotated on the head's first rd entries with the table (rd / 2
// a multiple of four), norm factors applied first (w may be null)
template <typename IT>
LWC_DEVICE float4v rotate4(const IT* src, int i, int rd, const float* tab, const float* w, float rstd) {
  float4v x = Vec4<IT>::ld(src + i);
  if (w) x *= Vec4<float>::ld(w + i) * rstd;
  if (i < rd) {
    const int half = rd >> 1;
    const bool first = i < half;
    const int m = first ? i : i - half, j = first ? i + half : i - half;
    float4v xp = Vec4<IT>::ld(src + j);
    if (w) xp *= Vec4<float>::ld(w + j) * rstd;
    const float4v cs = Vec4<float>::ld(tab + m), sn = Vec4<float>::ld(tab + half + m);
    x = first ? x * cs - xp * sn : x * cs + xp * sn;
  }
  return x;
}

// D, Dv multiples of four, rd and (rotated) Dv multiples of eight, every base a multiple of four entries: the angles
// of a row are formed once for all heads, 8- / 16-byte accesses except the interleaved value stores.
template <typename IT, typename CT>
__global__ void __launch_bounds__(256) rot_kv_write_vec_kernel(
    const IT* __restrict__ src, int lds, const float* __restrict__ wq, const float* __restrict__ wk,
    const float* __restrict__ freq, float mult, int rd, const float* __restrict__ vfreq, const int* __restrict__ positions,
    const int* __restrict__ slots, float* __restrict__ q_out, CT* __restrict__ k_cache, CT* __restrict__ v_cache,
    long long kb_stride, long long vb_stride, int block_size, int H, int G, int D, int Dv, float eps, float scale) {
  extern __shared__ __attribute__((aligned(16))) float sh[];  // [rd] angles of q / k | [Dv] angles of v | [H + G] norm factors
  float* tab = sh;
  float* vtab = sh + rd;
  float* rstd_s = vtab + (vfreq ? Dv : 0);
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const IT* pr = src + (size_t)t * lds;
  const float pos = (float)positions[t];
  const int slot = slots[t];
  const bool write = slot >= 0;
  const long long blk = write ? slot / block_size : 0, off = write ? slot % block_size : 0;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  if (rd) angle_table(tab, freq, rd >> 1, mult, pos);
  if (vfreq) angle_table(vtab, vfreq, Dv >> 1, 1.0f, pos);
  // D / 4 a power of two up to 64: the D / 4 threads that share a head in the loop below are neighbours in one wave
  // and sum its squares among themselves; else one wave per head beforehand
  const int d4 = D >> 2, dv4 = Dv >> 2;
  const bool among = wq && d4 <= 64 && (d4 & (d4 - 1)) == 0;
  if (wq && !among) {
    for (int h = wv; h < H + G; h += nw) {
      const IT* x = pr + (size_t)h * D;  // the k heads follow the q heads
      float s = 0.f;
      for (int i = lane * 4; i < D; i += 256) {
        const float4v v = Vec4<IT>::ld(x + i);
        s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
      }
      s = wave_sum(s);
      if (lane == 0) rstd_s[h] = 1.0f / sqrtf(s / (float)D + eps);
    }
  }
  __syncthreads();
  const int uq = H * d4, uk = write ? G * d4 : 0, uv = write ? G * dv4 : 0;
  for (int u = threadIdx.x; u < uq + uk + uv; u += blockDim.x) {
    if (u < uq + uk) {
      const int h = u / d4, i = (u - h * d4) * 4;  // h < H: a query head, else key head h - H
      float rstd = 1.0f;
      if (among) {
        const float4v v = Vec4<IT>::ld(pr + (size_t)h * D + i);
        float sq = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        for (int m = d4 >> 1; m > 0; m >>= 1) sq += __shfl_xor(sq, m, 64);
        rstd = 1.0f / sqrtf(sq / (float)D + eps);
      } else if (wq) {
        rstd = rstd_s[h];
      }
      const float4v x = rotate4<IT>(pr + (size_t)h * D, i, rd, tab, h < H ? wq : wk, rstd);
      if (h < H) Vec4<float>::st(q_out + (size_t)t * nq + (size_t)h * D + i, x * scale);
      else Vec4<CT>::st(k_cache + blk * kb_stride + off * nk + (size_t)(h - H) * D + i, x);
    } else {
      const int e = u - uq - uk, g = e / dv4, i = (e - g * dv4) * 4;
      const float4v x = rotate4<IT>(pr + nq + nk + (size_t)g * Dv, i, vfreq ? Dv : 0, vtab, nullptr, 1.0f);
      // V is 4-token interleaved: [block][offset / 4][column][offset % 4]
      CT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3) + 4LL * (g * Dv + i);
#pragma unroll
      for (int c = 0; c < 4; ++c) Elem<CT>::st(vc + 4 * c, x[c]);
    }
  }
}

template <typename AT>
__global__ void __launch_bounds__(256) head_gate_unrotate_vec_kernel(const AT* __restrict__ o, int ldi, const AT* __restrict__ g,
                                                                      int ldg, const float* __restrict__ vfreq,
                                                                      const int* __restrict__ positions, AT* __restrict__ out,
                                                                      int ldo, int H, int Dv, float scale) {
  extern __shared__ __attribute__((aligned(16))) float sh[];  // [Dv] angles
  const int t = blockIdx.x;
  if (vfreq) angle_table(sh, vfreq, Dv >> 1, 1.0f, -(float)positions[t]);  // turned back: the angles' signs flip
  __syncthreads();
  const int dv4 = Dv >> 2;
  for (int u = threadIdx.x; u < H * dv4; u += blockDim.x) {
    const int h = u / dv4, i = (u - h * dv4) * 4;
    const float gate = scale * (g ? sigmoid_f(Elem<AT>::ld(g + (size_t)t * ldg + h)) : 1.0f);
    const float4v x = rotate4<AT>(o + (size_t)t * ldi + (size_t)h * Dv, i, vfreq ? Dv : 0, sh, nullptr, 1.0f);
    Vec4<AT>::st(out + (size_t)t * ldo + (size_t)h * Dv + i, x * gate);
  }
}

template <typename YT, typename OT>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const YT* __restrict__ y, int ldy, const float* __restrict__ w,
                                   OT* __restrict__ out, int ldo, int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * d;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float v = xr[i] + (y ? Elem<YT>::ld(y + (size_t)t * ldy + i) : 0.f);
    if (y) xr[i] = v;
    s += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) Elem<OT>::st(out + (size_t)t * ldo + i, xr[i] * rstd * w[i]);
}

// rows of d <= 4 * 256 * NCH entries, every base a multiple of four: the new x stays in registers between the sum and
// the norm; 16-byte accesses
template <typename YT, typename OT, int NCH>
__global__ void __launch_bounds__(256) add_rmsnorm_vec_kernel(float* __restrict__ x, const YT* __restrict__ y, int ldy,
                                                               const float* __restrict__ w, OT* __restrict__ out, int ldo,
                                                               int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * d;
  float4v v[NCH];
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    v[u] = float4v{0.f, 0.f, 0.f, 0.f};
    if (i < d) {
      v[u] = Vec4<float>::ld(xr + i);
      if (y) {
        v[u] += Vec4<YT>::ld(y + (size_t)t * ldy + i);
        Vec4<float>::st(xr + i, v[u]);
      }
      s += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(s, scratch) / (float)d + eps);
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    if (i < d) Vec4<OT>::st(out + (size_t)t * ldo + i, v[u] * rstd * Vec4<float>::ld(w + i));
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

// io: bit 0 = rows fp32 (else bf16), bit 1 = cache fp32 (else bf16).  wq / wk / vfreq may be null; freq may be null
// when rd == 0.
extern "C" int r32_rot_kv_write(const void* src, int lds, const float* wq, const float* wk, const float* freq, float mult,
                                int rd, const float* vfreq, const int* positions, const int* slots, float* q_out,
                                void* k_cache, void* v_cache, long long kb_stride, long long vb_stride, int block_size, int T,
                                int H, int G, int D, int Dv, float eps, float scale, int io, hipStream_t s) {
  if (T <= 0) return 0;
  if (rd < 0 || rd > D || (rd & 1) || (rd > 0 && !freq) || (vfreq && (Dv & 1))) return -1;
  const int ib = (io & 1) ? 16 : 8, cb = (io & 2) ? 16 : 8;
  const bool vec = D % 4 == 0 && Dv % 4 == 0 && rd % 8 == 0 && (!vfreq || Dv % 8 == 0) && lds % 4 == 0 && kb_stride % 4 == 0 &&
                   (!wq == !wk) && aligned_to(src, ib) && aligned_to(k_cache, cb) && aligned_to(q_out, 16) &&
                   aligned_to(wq, 16) && aligned_to(wk, 16);
  const size_t shm = (size_t)(rd + (vfreq ? Dv : 0) + H + G) * sizeof(float);
#define LWC_ROT(IT, CT)                                                                                                \
  if (vec)                                                                                                             \
    rot_kv_write_vec_kernel<IT, CT><<<T, 256, shm, s>>>((const IT*)src, lds, wq, wk, freq, mult, rd, vfreq, positions, \
                                                        slots, q_out, (CT*)k_cache, (CT*)v_cache, kb_stride, vb_stride, \
                                                        block_size, H, G, D, Dv, eps, scale);                           \
  else                                                                                                                 \
    rot_kv_write_kernel<IT, CT><<<T, 256, 0, s>>>((const IT*)src, lds, wq, wk, freq, mult, rd, vfreq, positions, slots, \
                                                  q_out, (CT*)k_cache, (CT*)v_cache, kb_stride, vb_stride, block_size,  \
                                                  H, G, D, Dv, eps, scale)
  if (io == 3) {
    LWC_ROT(float, float);
  } else if (io == 0) {
    LWC_ROT(bf16_t, bf16_t);
  } else if (io == 1) {
    LWC_ROT(float, bf16_t);
  } else {
    return -1;
  }
#undef LWC_ROT
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_head_gate_unrotate(const void* o, int ldi, const void* g, int ldg, const float* vfreq,
                                      const int* positions, void* out, int ldo, int T, int H, int Dv, float scale, int f32,
                                      hipStream_t s) {
  if (T <= 0) return 0;
  if (vfreq && (Dv & 1)) return -1;
  const int threads = H >= 4 ? 256 : 64 * H;
  const int ab = f32 ? 16 : 8;
  if (Dv % 4 == 0 && (!vfreq || Dv % 8 == 0) && ldi % 4 == 0 && ldo % 4 == 0 && aligned_to(o, ab) && aligned_to(out, ab)) {
    const size_t shm = (size_t)(vfreq ? Dv : 4) * sizeof(float);
    if (f32)
      head_gate_unrotate_vec_kernel<float><<<T, 256, shm, s>>>((const float*)o, ldi, (const float*)g, ldg, vfreq, positions,
                                                                (float*)out, ldo, H, Dv, scale);
    else
      head_gate_unrotate_vec_kernel<bf16_t><<<T, 256, shm, s>>>((const bf16_t*)o, ldi, (const bf16_t*)g, ldg, vfreq,
                                                                 positions, (bf16_t*)out, ldo, H, Dv, scale);
    LWC_CHECK_LAUNCH();
    return 0;
  }
  if (f32)
    head_gate_unrotate_kernel<float><<<T, threads, 0, s>>>((const float*)o, ldi, (const float*)g, ldg, vfreq, positions,
                                                            (float*)out, ldo, H, Dv, scale);
  else
    head_gate_unrotate_kernel<bf16_t><<<T, threads, 0, s>>>((const bf16_t*)o, ldi, (const bf16_t*)g, ldg, vfreq, positions,
                                                             (bf16_t*)out, ldo, H, Dv, scale);
  LWC_CHECK_LAUNCH();
  return 0;
}

// y may be null (norm only); io: bit 0 = y fp32, bit 1 = out fp32
extern "C" int r32_add_rmsnorm(float* x, const void* y, int ldy, const float* w, void* out, int ldo, int T, int d, float eps,
                               int io, hipStream_t s) {
  if (T <= 0) return 0;
  const bool yf = io & 1, of = io & 2;
  const bool vec = d % 4 == 0 && d <= 8192 && ldy % 4 == 0 && ldo % 4 == 0 && aligned_to(x, 16) && aligned_to(w, 16) &&
                   aligned_to(y, yf ? 16 : 8) && aligned_to(out, of ? 16 : 8);
  const int nch = (d + 1023) / 1024;
#define LWC_ARN(YT, OT)                                                                                              \
  if (!vec) add_rmsnorm_kernel<YT, OT><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, w, (OT*)out, ldo, d, eps);           \
  else if (nch <= 1) add_rmsnorm_vec_kernel<YT, OT, 1><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, w, (OT*)out, ldo, d, eps); \
  else if (nch <= 2) add_rmsnorm_vec_kernel<YT, OT, 2><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, w, (OT*)out, ldo, d, eps); \
  else if (nch <= 4) add_rmsnorm_vec_kernel<YT, OT, 4><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, w, (OT*)out, ldo, d, eps); \
  else add_rmsnorm_vec_kernel<YT, OT, 8><<<T, 256, 0, s>>>(x, (const YT*)y, ldy, w, (OT*)out, ldo, d, eps)
  if (yf && of) {
    LWC_ARN(float, float);
  } else if (yf) {
    LWC_ARN(float, bf16_t);
  } else if (of) {
    LWC_ARN(bf16_t, float);
  } else {
    LWC_ARN(bf16_t, bf16_t);
  }
#undef LWC_ARN
  LWC_CHECK_LAUNCH();
  return 0;
}

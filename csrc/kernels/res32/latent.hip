// Low-rank ("latent") attention: what surrounds the attention kernels (gfx950, wave64).
//
// Queries and keys / values go through small latents.  Per token the cache holds ONE key row for all heads,
//   K = [ c (C entries, RMS-normalised latent) | rotated key part (R entries) | zeros up to the row size ]
// and V = c once more in the cache's 4-token interleaved value layout (zeros up to its row size).  With the keys'
// and values' up-projections moved to the query and to the attention's result, every head is a query head over that
// one row (key size C + R, value size C), which the window_attn kernels run with G = 1.
//
//   latent_kv_write   from fused projection rows [ dq (Cq) | dkv (C + R) | ... ]: cq = dq / rms(dq) * wq -> rows of the
//                     activation type; c = dkv[:C] / rms * wc and the rotated rest -> the paged cache
//   latent_q_rows     the fp32 query rows [ qn * scale (C) | rot(q_rot) * scale (R) | 0 ] per head from the absorbed
//                     unrotated part qn ([H, T, C] fp32) and the up-projected query rows (rotated part of every head)
//
// Rotation ("interleaved"): entries (2i, 2i + 1) at position p turn by the angle a = p * f_i (fp32 product of the
// position and the fp32 frequency), (u, v) -> m (u cos a - v sin a, v cos a + u sin a); f and m come from the host
// (frequency blending and the table multiplier of a scaled rotation are folded in there).
#include "elem.h"

namespace lwc {
namespace {

template <typename AT>
__global__ void __launch_bounds__(256)
latent_kv_write_kernel(const AT* __restrict__ proj, int ldp, int Cq, int C, int R, const float* __restrict__ wq,
                       const float* __restrict__ wc, const float* __restrict__ freq, float mult,
                       const int* __restrict__ positions, const int* __restrict__ slots, AT* __restrict__ cq, int ldq,
                       AT* __restrict__ k_cache, AT* __restrict__ v_cache, long long kb_stride, long long vb_stride,
                       int block_size, int nk, int nv, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const AT* pr = proj + (size_t)t * ldp;
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < Cq; i += blockDim.x) {
    const float x = Elem<AT>::ld(pr + i);
    sq += x * x;
  }
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const float x = Elem<AT>::ld(pr + Cq + i);
    sc += x * x;
  }
  const float rq = 1.0f / sqrtf(block_sum(sq, scratch) / (float)Cq + eps);
  const float rc = 1.0f / sqrtf(block_sum(sc, scratch) / (float)C + eps);
  for (int i = threadIdx.x; i < Cq; i += blockDim.x)
    Elem<AT>::st(cq + (size_t)t * ldq + i, Elem<AT>::ld(pr + i) * rq * wq[i]);
  const int slot = slots[t];
  if (slot < 0) return;
  const long long blk = slot / block_size, off = slot % block_size;
  AT* kc = k_cache + blk * kb_stride + off * nk;
  AT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * nv) + (off & 3);  // [offset / 4][column][offset % 4]
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const float c = Elem<AT>::ld(pr + Cq + i) * rc * wc[i];
    Elem<AT>::st(kc + i, c);
    Elem<AT>::st(vc + 4 * i, c);
  }
  const float p = (float)positions[t];
  for (int i = threadIdx.x; i < R / 2; i += blockDim.x) {
    const float a = p * freq[i];
    float sn, cs;
    sincosf(a, &sn, &cs);
    const float u = Elem<AT>::ld(pr + Cq + C + 2 * i), v = Elem<AT>::ld(pr + Cq + C + 2 * i + 1);
    Elem<AT>::st(kc + C + 2 * i, (u * cs - v * sn) * mult);
    Elem<AT>::st(kc + C + 2 * i + 1, (v * cs + u * sn) * mult);
  }
  for (int i = C + R + threadIdx.x; i < nk; i += blockDim.x) Elem<AT>::st(kc + i, 0.f);
  for (int i = C + threadIdx.x; i < nv; i += blockDim.x) Elem<AT>::st(vc + 4 * i, 0.f);
}

// q rows [T, H * (D + R)] (only the rotated part, columns D .. D + R of every head, is read); qn fp32 [H, T, C];
// out fp32 [T, H, Dk], Dk >= C + R
template <typename AT>
__global__ void __launch_bounds__(256)
latent_q_rows_kernel(const AT* __restrict__ q, int ldq, int D, int R, const float* __restrict__ qn, int C,
                     const float* __restrict__ freq, float mult, float scale, const int* __restrict__ positions,
                     float* __restrict__ out, int H, int Dk, int T) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  float* o = out + (size_t)t * H * Dk;
  for (int e = threadIdx.x; e < H * C; e += blockDim.x) {
    const int h = e / C, i = e - h * C;
    // without qn the unrotated part is the row's own (C == D then)
    o[(size_t)h * Dk + i] = (qn ? qn[((size_t)h * T + t) * C + i] : Elem<AT>::ld(q + (size_t)t * ldq + (size_t)h * (D + R) + i)) * scale;
  }
  for (int e = threadIdx.x; e < H * (R / 2); e += blockDim.x) {
    const int h = e / (R / 2), i = e - h * (R / 2);
    const float a = p * freq[i];
    float sn, cs;
    sincosf(a, &sn, &cs);
    const AT* qr = q + (size_t)t * ldq + (size_t)h * (D + R) + D;
    const float u = Elem<AT>::ld(qr + 2 * i), v = Elem<AT>::ld(qr + 2 * i + 1);
    o[(size_t)h * Dk + C + 2 * i] = (u * cs - v * sn) * (mult * scale);
    o[(size_t)h * Dk + C + 2 * i + 1] = (v * cs + u * sn) * (mult * scale);
  }
  const int pad = Dk - C - R;
  for (int e = threadIdx.x; e < H * pad; e += blockDim.x) {
    const int h = e / pad, i = e - h * pad;
    o[(size_t)h * Dk + C + R + i] = 0.f;
  }
}

// One workgroup per token: key rows [H][dk] = [kv key of the head (D) | the token's rotated part (R) | 0], value rows
// [H][dv] = [kv value | 0] in the 4-token interleaved layout.
template <typename AT>
__global__ void __launch_bounds__(256)
latent_expand_write_kernel(const AT* __restrict__ kv, int ldk, const AT* __restrict__ lat, int ldl, int rot_off,
                           const long long* __restrict__ slots, AT* __restrict__ k_cache, AT* __restrict__ v_cache,
                           long long kb_stride, long long vb_stride, int block_size, int H, int D, int R, int Dv, int dk, int dv) {
  const int t = blockIdx.x;
  const long long slot = slots[t];
  if (slot < 0) return;
  const long long blk = slot / block_size, off = slot % block_size;
  const AT* kr = kv + (size_t)t * ldk;
  const AT* lr = lat + (size_t)t * ldl + rot_off;
  AT* kc = k_cache + blk * kb_stride + off * ((long long)H * dk);
  AT* vc = v_cache + blk * vb_stride + (off >> 2) * (4LL * H * dv) + (off & 3);
  for (int e = threadIdx.x; e < H * dk; e += blockDim.x) {
    const int h = e / dk, i = e - h * dk;
    AT v = 0;
    if (i < D) v = kr[h * D + i];
    else if (i < D + R) v = lr[i - D];
    kc[e] = v;
  }
  for (int e = threadIdx.x; e < H * dv; e += blockDim.x) {
    const int h = e / dv, i = e - h * dv;
    vc[4 * e] = i < Dv ? kr[H * D + h * Dv + i] : (AT)0;
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_latent_expand_write(const void* kv, int ldk, const void* lat, int ldl, int rot_off, const long long* slots,
                                       void* k_cache, void* v_cache, long long kb_stride, long long vb_stride, int block_size,
                                       int N, int H, int D, int R, int Dv, int dk, int dv, int f32, hipStream_t s) {
  if (N <= 0) return 0;
  if (dk < D + R || dv < Dv) return -1;
  if (f32)
    latent_expand_write_kernel<float><<<N, 256, 0, s>>>((const float*)kv, ldk, (const float*)lat, ldl, rot_off, slots,
                                                        (float*)k_cache, (float*)v_cache, kb_stride, vb_stride, block_size, H, D,
                                                        R, Dv, dk, dv);
  else
    latent_expand_write_kernel<bf16_t><<<N, 256, 0, s>>>((const bf16_t*)kv, ldk, (const bf16_t*)lat, ldl, rot_off, slots,
                                                         (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride, vb_stride, block_size,
                                                         H, D, R, Dv, dk, dv);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_latent_kv_write(const void* proj, int ldp, int Cq, int C, int R, const float* wq, const float* wc,
                                   const float* freq, float mult, const int* positions, const int* slots, void* cq, int ldq,
                                   void* k_cache, void* v_cache, long long kb_stride, long long vb_stride, int block_size,
                                   int nk, int nv, float eps, int T, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (R % 2 != 0 || nk < C + R || nv < C || Cq < 1 || C < 1) return -1;
  if (f32)
    latent_kv_write_kernel<float><<<T, 256, 0, s>>>((const float*)proj, ldp, Cq, C, R, wq, wc, freq, mult, positions, slots,
                                                    (float*)cq, ldq, (float*)k_cache, (float*)v_cache, kb_stride, vb_stride,
                                                    block_size, nk, nv, eps);
  else
    latent_kv_write_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)proj, ldp, Cq, C, R, wq, wc, freq, mult, positions,
                                                     slots, (bf16_t*)cq, ldq, (bf16_t*)k_cache, (bf16_t*)v_cache, kb_stride,
                                                     vb_stride, block_size, nk, nv, eps);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_latent_q_rows(const void* q, int ldq, int D, int R, const float* qn, int C, const float* freq, float mult,
                                 float scale, const int* positions, float* out, int H, int Dk, int T, int f32,
                                 hipStream_t s) {
  if (T <= 0) return 0;
  if (R % 2 != 0 || Dk < C + R) return -1;
  if (f32)
    latent_q_rows_kernel<float><<<T, 256, 0, s>>>((const float*)q, ldq, D, R, qn, C, freq, mult, scale, positions, out, H, Dk, T);
  else
    latent_q_rows_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)q, ldq, D, R, qn, C, freq, mult, scale, positions, out, H, Dk, T);
  LWC_CHECK_LAUNCH();
  return 0;
}

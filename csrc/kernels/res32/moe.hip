// Mixture-of-experts routing with a softmax router over real and identity experts (gfx950, wave64).
//
//   router_topk     s = softmax(z) over all NE router outputs (fp32); the k largest of s + correction are chosen
//                   (ties: the lower index); the weights are the chosen s, not renormalised.  Outputs beyond the
//                   first E are IDENTITY experts (their output is the token's input itself).  Counts the rows of
//                   every real expert and hands each (token, choice) its rank within its expert.
//   router_offsets  exclusive scan of the counts -> row_off [E + 1]
//   router_scatter  expert-major rows: src[row] = token, row_expert[row], inv[t*k + j] = row (-1: identity)
//   expert_rows     one workgroup per expert-major row: y = W_down (silu(W_gate h) * (W_up h)), any sizes, fp32 sums
//   moe_combine     out[t] = sum_j w[t][j] * (inv >= 0 ? Y[inv] : h[t])   (fp32)
#include "elem.h"

namespace lwc {
namespace {

constexpr int kMaxPerLane = 8;  // router outputs per lane: NE <= 512

template <int PER>
__global__ void router_topk_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                   const float* __restrict__ bias, int renorm, int NE, int E, int k,
                                   int* __restrict__ ids, float* __restrict__ wts, int* __restrict__ counts,
                                   int* __restrict__ rank, int T) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= T) return;
  const int lane = threadIdx.x & 63;
  const float* zr = z + (size_t)t * NE;
  float v[PER], c[PER];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < NE ? zr[e] + (bias ? bias[e] : 0.f) : -INFINITY;
    m = fmaxf(m, v[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < NE ? expf(v[i] - m) : 0.f;
    sum += v[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + 64 * i;
    v[i] = v[i] / sum;
    c[i] = e < NE ? v[i] + (corr ? corr[e] : 0.f) : -INFINITY;
  }
  float chosen = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + 64 * i;
      if (e < NE && (c[i] > best || (c[i] == best && e < bi))) best = c[i], bi = e;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) best = ob, bi = oi;
    }
    // the winner's lane removes it and reports its score
    float sc = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (lane + 64 * i == bi) sc = v[i], c[i] = -INFINITY;
    sc = wave_sum(sc);
    chosen += sc;
    if (lane == 0) {
      ids[(size_t)t * k + j] = bi;
      wts[(size_t)t * k + j] = sc;
      rank[(size_t)t * k + j] = bi < E ? atomicAdd(counts + bi, 1) : -1;
    }
  }
  if (renorm && lane == 0)  // weights = softmax over the chosen outputs only
    for (int j = 0; j < k; ++j) wts[(size_t)t * k + j] /= chosen;
}

// Few router outputs (NE <= NMAX): one THREAD per token, the scores in registers.
template <int NMAX>
__global__ void router_topk_thread_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                          const float* __restrict__ bias, int renorm, int NE, int E, int k,
                                          int* __restrict__ ids, float* __restrict__ wts, int* __restrict__ counts,
                                          int* __restrict__ rank, int T) {
  const int t0 = blockIdx.x * blockDim.x + threadIdx.x;
  const bool live = t0 < T;  // lanes past the last token go along (wave-wide votes below) and write nothing
  const int t = live ? t0 : T - 1;
  const float* zr = z + (size_t)t * NE;
  float v[NMAX], c[NMAX];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NMAX; ++i) {
    v[i] = i < NE ? zr[i] + (bias ? bias[i] : 0.f) : -INFINITY;
    m = fmaxf(m, v[i]);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NMAX; ++i) {
    v[i] = i < NE ? expf(v[i] - m) : 0.f;
    sum += v[i];
  }
#pragma unroll
  for (int i = 0; i < NMAX; ++i) {
    v[i] = v[i] / sum;
    c[i] = i < NE ? v[i] + (corr ? corr[i] : 0.f) : -INFINITY;
  }
  float chosen = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY, sc = 0.f;
    int bi = 0;
#pragma unroll
    for (int i = 0; i < NMAX; ++i)
      if (i < NE && c[i] > best) best = c[i], bi = i, sc = v[i];
#pragma unroll
    for (int i = 0; i < NMAX; ++i)
      if (i == bi) c[i] = -INFINITY;
    chosen += sc;
    if (live) {
      ids[(size_t)t * k + j] = bi;
      wts[(size_t)t * k + j] = sc;
    }
    // one atomic per (wave, expert) instead of one per token: the wave's tokens that chose expert e take
    // consecutive ranks in lane order
    int rk = -1;
    for (int e = 0; e < E; ++e) {
      const unsigned long long m = __ballot(live && bi == e);
      if (m == 0ull) continue;
      const int leader = __ffsll((long long)m) - 1;
      int base = 0;
      if ((int)(threadIdx.x & 63) == leader) base = atomicAdd(counts + e, __popcll(m));
      base = __shfl(base, leader, 64);
      if (live && bi == e) rk = base + __popcll(m & ((1ull << (threadIdx.x & 63)) - 1ull));
    }
    if (live) rank[(size_t)t * k + j] = rk;
  }
  if (renorm && live)  // weights = softmax over the chosen outputs only
    for (int j = 0; j < k; ++j) wts[(size_t)t * k + j] /= chosen;
}

__global__ void router_offsets_kernel(const int* __restrict__ counts, int E, int* __restrict__ row_off) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int o = 0;
    for (int e = 0; e < E; ++e) {
      row_off[e] = o;
      o += counts[e];
    }
    row_off[E] = o;
  }
}

__global__ void router_scatter_kernel(const int* __restrict__ ids, const int* __restrict__ rank,
                                      const int* __restrict__ row_off, int E, int k, int* __restrict__ src,
                                      int* __restrict__ row_expert, int* __restrict__ inv, int total) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int x = ids[e];
  if (x < E) {
    const int row = row_off[x] + rank[e];
    src[row] = e / k;
    row_expert[row] = x;
    inv[e] = row;
  } else {
    inv[e] = -1;
  }
}

// W_gu [E][2 ff][d]: gate rows then up rows; W_down [E][d][ff]
template <typename AT>
__global__ void __launch_bounds__(256) expert_rows_kernel(const AT* __restrict__ h, int ldh, const int* __restrict__ src,
                                                           const int* __restrict__ row_expert,
                                                           const int* __restrict__ row_off, int E,
                                                           const AT* __restrict__ w_gu, const AT* __restrict__ w_down,
                                                           float* __restrict__ Y, int d, int ff) {
  extern __shared__ float smem[];  // h [d] | act [ff]
  const int row = blockIdx.x;
  if (row >= row_off[E]) return;
  float* hs = smem;
  float* act = smem + d;
  const int t = src[row], e = row_expert[row];
  for (int i = threadIdx.x; i < d; i += blockDim.x) hs[i] = Elem<AT>::ld(h + (size_t)t * ldh + i);
  __syncthreads();
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const AT* wg = w_gu + (size_t)e * 2 * ff * d;
  for (int f = wv; f < ff; f += nw) {
    const AT* g = wg + (size_t)f * d;
    const AT* u = wg + (size_t)(ff + f) * d;
    float sg = 0.f, su = 0.f;
    for (int i = lane; i < d; i += 64) {
      sg += Elem<AT>::ld(g + i) * hs[i];
      su += Elem<AT>::ld(u + i) * hs[i];
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) act[f] = silu_f(sg) * su;
  }
  __syncthreads();
  const AT* wd = w_down + (size_t)e * d * ff;
  for (int c = wv; c < d; c += nw) {
    const AT* r = wd + (size_t)c * ff;
    float s = 0.f;
    for (int i = lane; i < ff; i += 64) s += Elem<AT>::ld(r + i) * act[i];
    s = wave_sum(s);
    if (lane == 0) Y[(size_t)row * d + c] = s;
  }
}

template <typename AT, typename YT>
__global__ void moe_combine_kernel(const YT* __restrict__ Y, const int* __restrict__ inv, const float* __restrict__ wts,
                                   const AT* __restrict__ h, int ldh, int k, float* __restrict__ out, int d,
                                   const AT* __restrict__ add, int lda) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float s = add ? Elem<AT>::ld(add + (size_t)t * lda + c) : 0.f;
    for (int j = 0; j < k; ++j) {
      const int r = inv[(size_t)t * k + j];
      const float v = r >= 0 ? Elem<YT>::ld(Y + (size_t)r * d + c) : Elem<AT>::ld(h + (size_t)t * ldh + c);
      s += wts[(size_t)t * k + j] * v;
    }
    out[(size_t)t * d + c] = s;
  }
}

// four columns per thread (d a multiple of four, aligned bases)
template <typename AT, typename YT>
__global__ void moe_combine_vec_kernel(const YT* __restrict__ Y, const int* __restrict__ inv, const float* __restrict__ wts,
                                       const AT* __restrict__ h, int ldh, int k, float* __restrict__ out, int d,
                                       const AT* __restrict__ add, int lda) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x * 4; c < d; c += blockDim.x * 4) {
    float4v s = add ? Vec4<AT>::ld(add + (size_t)t * lda + c) : float4v{0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const int r = inv[(size_t)t * k + j];
      const float4v v = r >= 0 ? Vec4<YT>::ld(Y + (size_t)r * d + c) : Vec4<AT>::ld(h + (size_t)t * ldh + c);
      s += v * wts[(size_t)t * k + j];
    }
    Vec4<float>::st(out + (size_t)t * d + c, s);
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_router_max_outputs() { return 64 * kMaxPerLane; }

// counts must be zero on entry (E ints)
// corr (added to the softmax for the choice only) and bias (added to the logits) may be null; renorm != 0: the chosen
// weights are divided by their sum
extern "C" int r32_router(const float* z, const float* corr, const float* bias, int renorm, int T, int NE, int E, int k,
                          int* ids, float* wts, int* counts, int* rank, int* row_off, int* src, int* row_expert, int* inv,
                          hipStream_t s) {
  if (T <= 0) return 0;
  if (NE > 64 * kMaxPerLane || k < 1 || k > NE || E > NE) return -1;
  if (NE <= 16) router_topk_thread_kernel<16><<<(T + 63) / 64, 64, 0, s>>>(z, corr, bias, renorm, NE, E, k, ids, wts, counts, rank, T);
  else if (NE <= 64) router_topk_kernel<1><<<(T + 3) / 4, 256, 0, s>>>(z, corr, bias, renorm, NE, E, k, ids, wts, counts, rank, T);
  else router_topk_kernel<kMaxPerLane><<<(T + 3) / 4, 256, 0, s>>>(z, corr, bias, renorm, NE, E, k, ids, wts, counts, rank, T);
  router_offsets_kernel<<<1, 64, 0, s>>>(counts, E, row_off);
  const int total = T * k;
  router_scatter_kernel<<<(total + 255) / 256, 256, 0, s>>>(ids, rank, row_off, E, k, src, row_expert, inv, total);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_expert_rows(const void* h, int ldh, const int* src, const int* row_expert, const int* row_off, int E,
                               const void* w_gu, const void* w_down, float* Y, int rows, int d, int ff, int f32,
                               hipStream_t s) {
  if (rows <= 0) return 0;
  const size_t shm = (size_t)(d + ff) * sizeof(float);
  if (shm > 60000) return -1;
  if (f32)
    expert_rows_kernel<float><<<rows, 256, shm, s>>>((const float*)h, ldh, src, row_expert, row_off, E, (const float*)w_gu,
                                                      (const float*)w_down, Y, d, ff);
  else
    expert_rows_kernel<bf16_t><<<rows, 256, shm, s>>>((const bf16_t*)h, ldh, src, row_expert, row_off, E, (const bf16_t*)w_gu,
                                                       (const bf16_t*)w_down, Y, d, ff);
  LWC_CHECK_LAUNCH();
  return 0;
}

// add: rows of the activation type added to every token's sum (a shared expert), or null
extern "C" int r32_moe_combine(const void* Y, int y_f32, const int* inv, const float* wts, const void* h, int ldh, int T,
                               int k, float* out, int d, const void* add, int lda, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (d % 4 == 0 && ldh % 4 == 0 && lda % 4 == 0 && aligned_to(add, f32 ? 16 : 8) && aligned_to(Y, y_f32 ? 16 : 8) && aligned_to(h, f32 ? 16 : 8) && aligned_to(out, 16)) {
    if (f32 && y_f32)
      moe_combine_vec_kernel<float, float><<<T, 256, 0, s>>>((const float*)Y, inv, wts, (const float*)h, ldh, k, out, d, (const float*)add, lda);
    else if (!f32 && y_f32)
      moe_combine_vec_kernel<bf16_t, float><<<T, 256, 0, s>>>((const float*)Y, inv, wts, (const bf16_t*)h, ldh, k, out, d, (const bf16_t*)add, lda);
    else if (!f32 && !y_f32)
      moe_combine_vec_kernel<bf16_t, bf16_t><<<T, 256, 0, s>>>((const bf16_t*)Y, inv, wts, (const bf16_t*)h, ldh, k, out, d, (const bf16_t*)add, lda);
    else
      return -1;
    LWC_CHECK_LAUNCH();
    return 0;
  }
  if (f32 && y_f32)
    moe_combine_kernel<float, float><<<T, 256, 0, s>>>((const float*)Y, inv, wts, (const float*)h, ldh, k, out, d, (const float*)add, lda);
  else if (!f32 && y_f32)
    moe_combine_kernel<bf16_t, float><<<T, 256, 0, s>>>((const float*)Y, inv, wts, (const bf16_t*)h, ldh, k, out, d, (const bf16_t*)add, lda);
  else if (!f32 && !y_f32)
    moe_combine_kernel<bf16_t, bf16_t><<<T, 256, 0, s>>>((const bf16_t*)Y, inv, wts, (const bf16_t*)h, ldh, k, out, d, (const bf16_t*)add, lda);
  else
    return -1;
  LWC_CHECK_LAUNCH();
  return 0;
}

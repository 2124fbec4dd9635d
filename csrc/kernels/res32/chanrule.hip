// Linear-attention recurrences with a decay per head AND key channel, over per-sequence state slots (gfx950, wave64).
//
// A step's rows are grouped in items as in recurrent.hip (rows of one sequence at consecutive positions + a state slot).
// Per head, with g_t a vector over the D key channels (it scales the ROWS of the D x Dv state):
//
//   DELTA = 0 (gated linear attention)   S <- diag(g_t) S + k_t v_t^T                      o_t = S^T q_t
//   DELTA = 1 (gated delta rule)         S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//
//   chan_prep   per row, in parallel over rows: rows [q (G*D) | k (G*D) | v (H*Dv)] -> fp32 (in place when they are
//               fp32 already); q, k made unit vectors per head (1e-6 inside the root) when asked; q times D^-1/2;
//               the decays from their logits z [T, H*D]:
//                 with A_log:   g = exp(-exp(A_log_h) softplus(z + zb))
//                 without:      g = sigmoid(z + zb)^(1/tau) = exp(-softplus(-(z + zb)) / tau)
//               beta = sigmoid(b_h) (or 1) and q . k per q/k head
//   chan_rule   the recurrence: the work split of delta_rule (a workgroup of NW waves per (item, head, 16 NW value
//               columns), a quarter state column per lane (an eighth, 8 NW columns, when the grid would leave SIMDs
//               with fewer than two waves), a token's k, q and g staged once through LDS,
//               double-buffered, loads five tokens ahead in straight-line code).  With Sg = g S (one multiply per state element):
//               S^T k and S^T q over Sg in one pass, o = Sg^T q + (k . q) u, S = Sg + k u^T.
#include "elem.h"

namespace lwc {
namespace {

template <typename ST, typename ZT, typename BT>
__global__ void chan_prep_kernel(const ST* __restrict__ src, int lds, float* __restrict__ qkv, int ldq,
                                 const ZT* __restrict__ z, int ldz, const float* __restrict__ zb,
                                 const float* __restrict__ A_log, float inv_tau, const BT* __restrict__ b, int ldb,
                                 float* __restrict__ dec, float* __restrict__ bq, int H, int G, int D, int Dv, int unit) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float qscale = 1.0f / sqrtf((float)D);
  const ST* sr = src + (size_t)t * lds;
  float* dr = qkv + (size_t)t * ldq;
  for (int v = wv; v < 2 * G; v += nw) {  // q heads, then k heads
    const ST* x = sr + (size_t)v * D;
    float* y = dr + (size_t)v * D;
    float r = v < G ? qscale : 1.0f;
    if (unit) {
      float s = 0.f;
      for (int i = lane; i < D; i += 64) {
        const float e = Elem<ST>::ld(x + i);
        s += e * e;
      }
      r /= sqrtf(wave_sum(s) + 1e-6f);
    }
    for (int i = lane; i < D; i += 64) y[i] = Elem<ST>::ld(x + i) * r;
  }
  if ((const void*)src != (const void*)qkv) {
    const int nv = H * Dv, o = 2 * G * D;
    for (int i = threadIdx.x; i < nv; i += blockDim.x) dr[o + i] = Elem<ST>::ld(sr + o + i);
  }
  const int nd = H * D;
  for (int e = threadIdx.x; e < nd; e += blockDim.x) {
    const float a = Elem<ZT>::ld(z + (size_t)t * ldz + e) + (zb ? zb[e] : 0.f);
    dec[(size_t)t * nd + e] = A_log ? expf(-expf(A_log[e / D]) * softplus_f(a)) : expf(-softplus_f(-a) * inv_tau);
  }
  const int nb = H + G;  // bq row: beta_h | (q . k)_g
  for (int h = threadIdx.x; h < H; h += blockDim.x)
    bq[(size_t)t * nb + h] = b ? sigmoid_f(Elem<BT>::ld(b + (size_t)t * ldb + h)) : 1.0f;
  __syncthreads();  // the fp32 q and k of this row are written
  for (int g = wv; g < G; g += nw) {
    const float* q = dr + (size_t)g * D;
    const float* k = q + (size_t)G * D;
    float s = 0.f;
    for (int i = lane; i < D; i += 64) s += q[i] * k[i];
    s = wave_sum(s);
    if (lane == 0) bq[(size_t)t * nb + H + g] = s;
  }
}

// D and Dv multiples of four, every base a multiple of four entries: 8- / 16-byte accesses
template <typename ST, typename ZT, typename BT>
__global__ void __launch_bounds__(256) chan_prep_vec_kernel(const ST* __restrict__ src, int lds, float* __restrict__ qkv, int ldq,
                                                             const ZT* __restrict__ z, int ldz, const float* __restrict__ zb,
                                                             const float* __restrict__ A_log, float inv_tau,
                                                             const BT* __restrict__ b, int ldb, float* __restrict__ dec,
                                                             float* __restrict__ bq, int H, int G, int D, int Dv, int unit) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float qscale = 1.0f / sqrtf((float)D);
  const ST* sr = src + (size_t)t * lds;
  float* dr = qkv + (size_t)t * ldq;
  const int nb = H + G;  // bq row: beta_h | (q . k)_g
  for (int g = wv; g < G; g += nw) {  // q and k of one q/k head: both norms and q . k from registers (D <= 256)
    const int i = lane * 4;
    float4v q = float4v{0.f, 0.f, 0.f, 0.f}, k = q;
    if (i < D) q = Vec4<ST>::ld(sr + (size_t)g * D + i), k = Vec4<ST>::ld(sr + (size_t)(G + g) * D + i);
    float rq = qscale, rk = 1.0f;
    if (unit) {
      rq /= sqrtf(wave_sum(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]) + 1e-6f);
      rk /= sqrtf(wave_sum(k[0] * k[0] + k[1] * k[1] + k[2] * k[2] + k[3] * k[3]) + 1e-6f);
    }
    q *= rq, k *= rk;
    const float qk = wave_sum(q[0] * k[0] + q[1] * k[1] + q[2] * k[2] + q[3] * k[3]);
    if (i < D) {
      Vec4<float>::st(dr + (size_t)g * D + i, q);
      Vec4<float>::st(dr + (size_t)(G + g) * D + i, k);
    }
    if (lane == 0) bq[(size_t)t * nb + H + g] = qk;
  }
  if ((const void*)src != (const void*)qkv) {
    const int nv = H * Dv, o = 2 * G * D;
    for (int i = threadIdx.x * 4; i < nv; i += blockDim.x * 4) Vec4<float>::st(dr + o + i, Vec4<ST>::ld(sr + o + i));
  }
  const int nd = H * D;
  for (int e = threadIdx.x * 4; e < nd; e += blockDim.x * 4) {
    float4v a = Vec4<ZT>::ld(z + (size_t)t * ldz + e);
    if (zb) a += Vec4<float>::ld(zb + e);
    float4v r;
    if (A_log) {
      const float rate = -expf(A_log[e / D]);
#pragma unroll
      for (int c = 0; c < 4; ++c) r[c] = expf(rate * softplus_f(a[c]));
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) r[c] = expf(-softplus_f(-a[c]) * inv_tau);
    }
    Vec4<float>::st(dec + (size_t)t * nd + e, r);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x)
    bq[(size_t)t * nb + h] = b ? sigmoid_f(Elem<BT>::ld(b + (size_t)t * ldb + h)) : 1.0f;
}

// RG lanes share a state column (RG = 4: 16 columns per wave; RG = 8: 8 columns per wave, twice the waves for small grids)
// ONE: every item is a single row (a decode step): nothing is fetched ahead and nothing staged for a next token.
template <int DPL, int NW, int DELTA, int RG, bool ONE>
__global__ void __launch_bounds__(64 * NW) chan_rule_kernel(const float* __restrict__ qkv, int ldq,
                                                             const float* __restrict__ dec, const float* __restrict__ bq,
                                                             float* __restrict__ state, long long slot_stride,
                                                             const int* __restrict__ cu, const int* __restrict__ item_slot,
                                                             const int* __restrict__ positions, float* __restrict__ out,
                                                             int ldo, int H, int G, int D, int Dv, int groups) {
  constexpr int QLD = DPL + 4;               // a row group's part in LDS, padded against bank conflicts
  constexpr int CW = 64 / RG;                // state columns per wave
  constexpr int PER = (3 * RG * DPL + 64 * NW - 1) / (64 * NW);  // staged floats per thread (k, q and g: 3 * RG DPL)
  __shared__ __attribute__((aligned(16))) float kqg_s[2][3][RG * QLD];  // [buffer][k | q | g][row groups]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, c = lane % CW, r = lane / CW;
  const int item = blockIdx.y, h = blockIdx.x / groups, grp = blockIdx.x - h * groups;
  const int col = (grp * NW + wv) * CW + c;
  const bool live = col < Dv;
  const int kvh = h / (H / G);
  const int r0 = cu[item], r1 = cu[item + 1];
  if (r1 <= r0) return;
  const int i0 = r * DPL;  // this lane's first state row
  float* Sg = state + (long long)item_slot[item] * slot_stride + ((size_t)h * D + i0) * Dv + col;
  float S[DPL];
  const bool fresh = positions[r0] == 0;
#pragma unroll
  for (int j = 0; j < DPL; ++j) S[j] = (i0 + j < D && live && !fresh) ? Sg[(size_t)j * Dv] : 0.f;
  const int nq = G * D, nd = H * D, nb = H + G;
  struct Stage {
    float kqg[PER], v, beta, qk;
  };
  auto fetch = [&](int row, Stage& st) {
    const float* qr = qkv + (size_t)row * ldq + kvh * D;
    const float* gr = dec + (size_t)row * nd + h * D;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 64 * NW * u;       // e / (RG DPL): 0 = k, 1 = q, 2 = g
      const int which = e / (RG * DPL), i = e - which * RG * DPL;
      float x = 0.f;
      if (e < 3 * RG * DPL && i < D) x = which == 0 ? qr[nq + i] : (which == 1 ? qr[i] : gr[i]);
      st.kqg[u] = x;
    }
    st.v = live ? qkv[(size_t)row * ldq + 2 * nq + h * Dv + col] : 0.f;
    st.beta = bq[(size_t)row * nb + h];
    st.qk = bq[(size_t)row * nb + H + kvh];
  };
  auto stash = [&](int buf, const Stage& st) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 64 * NW * u;
      const int which = e / (RG * DPL), i = e - which * RG * DPL;
      if (e < 3 * RG * DPL) kqg_s[buf][which][(i / DPL) * QLD + i % DPL] = st.kqg[u];
    }
  };
  auto group_sum = [](float x) {  // over the RG lanes of a column (lane bits 4, 5; with RG = 8 also bit 3)
    if (RG == 8) x += __shfl_xor(x, 8, 64);
    return row_sum4(x);
  };
  // Four register stages: a token's operands are fetched five tokens before its turn (a trip to memory takes about
  // as long as two tokens' arithmetic).  Every fetch is unconditional, past the item's end it repeats the last row, so
  // the loop body is straight-line code and the waits count exactly the loads still in flight.
  Stage st0, st1, st2, st3;
  const int rl = r1 - 1;
  fetch(r0, st0);
  stash(0, st0);
  float v = st0.v, beta = st0.beta, qk = st0.qk;
  if (!ONE) {
    fetch(min(r0 + 1, rl), st0);
    fetch(min(r0 + 2, rl), st1);
    fetch(min(r0 + 3, rl), st2);
    fetch(min(r0 + 4, rl), st3);
  }
  __syncthreads();
  auto step = [&](int row, int cur, Stage& next) {
    const float4v* ks = reinterpret_cast<const float4v*>(&kqg_s[cur][0][r * QLD]);
    const float4v* qs = reinterpret_cast<const float4v*>(&kqg_s[cur][1][r * QLD]);
    const float4v* gs = reinterpret_cast<const float4v*>(&kqg_s[cur][2][r * QLD]);
    float kk[DPL];
    float4v dk = float4v{0.f, 0.f, 0.f, 0.f}, dq = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < DPL / 4; ++j) {
      const float4v k4 = ks[j], q4 = qs[j], g4 = gs[j];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        kk[4 * j + e] = k4[e];
        S[4 * j + e] *= g4[e];
        if (DELTA) dk[e] += S[4 * j + e] * k4[e];
        dq[e] += S[4 * j + e] * q4[e];
      }
    }
    const float sq = group_sum((dq[0] + dq[1]) + (dq[2] + dq[3]));
    float u = v;
    if (DELTA) u = beta * (v - group_sum((dk[0] + dk[1]) + (dk[2] + dk[3])));
    if (live && r == 0) out[(size_t)row * ldo + h * Dv + col] = sq + qk * u;
#pragma unroll
    for (int j = 0; j < DPL; ++j) S[j] += kk[j] * u;
    if (ONE) return;
    stash(cur ^ 1, next);  // (behind the last token: a buffer nobody reads)
    v = next.v, beta = next.beta, qk = next.qk;
    fetch(min(row + 5, rl), next);
    __syncthreads();
  };
  int row = r0;
  if (ONE) {
    step(row, 0, st0);
    row = r1;
  }
  for (; row + 4 <= r1; row += 4) {
    step(row, 0, st0);
    step(row + 1, 1, st1);
    step(row + 2, 0, st2);
    step(row + 3, 1, st3);
  }
  if (row < r1) step(row, 0, st0);
  if (row + 1 < r1) step(row + 1, 1, st1);
  if (row + 2 < r1) step(row + 2, 0, st2);
  if (live) {
#pragma unroll
    for (int j = 0; j < DPL; ++j)
      if (i0 + j < D) Sg[(size_t)j * Dv] = S[j];
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_chan_rule_max_dim() { return 256; }

// src rows [q | k | v] (bf16 or fp32: src_f32) -> qkv fp32 (may be src itself); z decay logits (z_f32), zb fp32 [H D] or
// null, A_log fp32 [H] or null (then inv_tau), b beta logits [T, >= H] or null (b_f32); dec fp32 [T, H D] and bq fp32
// [T, H + G] scratch of the caller; state fp32 [slot][H][D][Dv]; out fp32 [T, H Dv].
extern "C" int r32_chan_rule(const void* src, int lds, int src_f32, float* qkv, int ldq, const void* z, int ldz, int z_f32,
                             const float* zb, const float* A_log, float inv_tau, const void* b, int ldb, int b_f32,
                             float* dec, float* bq, float* state, long long slot_stride, const int* cu,
                             const int* item_slot, const int* positions, float* out, int ldo, int T, int items, int H, int G,
                             int D, int Dv, int unit, int delta, hipStream_t s) {
  if (items <= 0 || T <= 0) return 0;
  if (D < 1 || D > 256 || G < 1 || H % G != 0) return -1;
  if (!src_f32 && (const void*)src == (const void*)qkv) return -1;
  const bool vec = D % 4 == 0 && Dv % 4 == 0 && lds % 4 == 0 && ldq % 4 == 0 && ldz % 4 == 0 && aligned_to(src, src_f32 ? 16 : 8) &&
                   aligned_to(qkv, 16) && aligned_to(z, z_f32 ? 16 : 8) && aligned_to(zb, 16);
#define LWC_PREP(ST, ZT, BT)                                                                                             \
  if (vec)                                                                                                               \
    chan_prep_vec_kernel<ST, ZT, BT><<<T, 256, 0, s>>>((const ST*)src, lds, qkv, ldq, (const ZT*)z, ldz, zb, A_log,     \
                                                       inv_tau, (const BT*)b, ldb, dec, bq, H, G, D, Dv, unit);         \
  else                                                                                                                   \
    chan_prep_kernel<ST, ZT, BT><<<T, 256, 0, s>>>((const ST*)src, lds, qkv, ldq, (const ZT*)z, ldz, zb, A_log, inv_tau, \
                                                   (const BT*)b, ldb, dec, bq, H, G, D, Dv, unit)
  if (b_f32 || !b) {
    if (src_f32 && z_f32) { LWC_PREP(float, float, float); }
    else if (src_f32) { LWC_PREP(float, bf16_t, float); }
    else if (z_f32) { LWC_PREP(bf16_t, float, float); }
    else { LWC_PREP(bf16_t, bf16_t, float); }
  } else {
    if (src_f32 && z_f32) { LWC_PREP(float, float, bf16_t); }
    else if (src_f32) { LWC_PREP(float, bf16_t, bf16_t); }
    else if (z_f32) { LWC_PREP(bf16_t, float, bf16_t); }
    else { LWC_PREP(bf16_t, bf16_t, bf16_t); }
  }
#undef LWC_PREP
  // A quarter column per lane; a grid that leaves SIMDs with fewer than two waves takes an eighth per lane instead
  // (twice the waves, half the arithmetic per lane and token: the recurrence is a chain of dependent steps per token).
  const long long waves4 = (long long)H * items * ((Dv + 15) / 16);
  const bool fine = waves4 < 2048 && D > 32;
  const int tiles = fine ? (Dv + 7) / 8 : (Dv + 15) / 16;
  const bool one = T == items;  // every item a single row
#define LWC_RULE_K(DPL, NW, DL, RG, ONE)                                                                            \
  chan_rule_kernel<DPL, NW, DL, RG, ONE><<<dim3(H * ((tiles + NW - 1) / NW), items), 64 * NW, 0, s>>>(              \
      qkv, ldq, dec, bq, state, slot_stride, cu, item_slot, positions, out, ldo, H, G, D, Dv, (tiles + NW - 1) / NW)
#define LWC_RULE(DPL, NW, RG)                 \
  if (delta && one) {                         \
    LWC_RULE_K(DPL, NW, 1, RG, true);         \
  } else if (delta) {                         \
    LWC_RULE_K(DPL, NW, 1, RG, false);        \
  } else if (one) {                           \
    LWC_RULE_K(DPL, NW, 0, RG, true);         \
  } else {                                    \
    LWC_RULE_K(DPL, NW, 0, RG, false);        \
  }
#define LWC_RULE_NW(DPL, RG)   \
  if (tiles >= 4) {            \
    LWC_RULE(DPL, 4, RG);      \
  } else if (tiles >= 2) {     \
    LWC_RULE(DPL, 2, RG);      \
  } else {                     \
    LWC_RULE(DPL, 1, RG);      \
  }
  if (fine) {
    if (D <= 64) {
      LWC_RULE_NW(8, 8)
    } else if (D <= 128) {
      LWC_RULE_NW(16, 8)
    } else {
      LWC_RULE_NW(32, 8)
    }
  } else if (D <= 32) {
    LWC_RULE_NW(8, 4)
  } else if (D <= 64) {
    LWC_RULE_NW(16, 4)
  } else if (D <= 128) {
    LWC_RULE_NW(32, 4)
  } else {
    LWC_RULE_NW(64, 4)
  }
#undef LWC_RULE_NW
#undef LWC_RULE
#undef LWC_RULE_K
  LWC_CHECK_LAUNCH();
  return 0;
}

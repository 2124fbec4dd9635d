// Recurrent mechanisms with per-sequence state slots (gfx950, wave64).
//
// A step's rows are grouped in ITEMS: item i owns rows [cu[i], cu[i+1]) of one sequence, consecutive positions
// (a decode row is an item of one row), and a state slot item_slot[i].  Nothing is read from a slot for a row
// whose history lies before position 0, so a slot needs no clearing when it is handed to a new sequence.
//
//   conv_hist         causal convolution over time per channel, y_t = sum_s w[c][taps-1-s] x_(t-s), s < taps; the
//                     inputs before the item's first row come from the slot's history (the last taps-1 inputs).
//                     MODE 0: out = x + y (and optionally a cast copy of x); MODE 1: out = silu(y); MODE 2: out = y
//   conv_hist_update  the slot's history after the step: the last taps-1 inputs of old history ++ this step's rows
//   delta_rule        gated delta rule, one wave per (item, head, 16 value columns), a quarter state column per lane:
//                       S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                     q, k made unit vectors per head (1e-6 inside the root), q times D^-1/2;
//                     beta = sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias)); state fp32 [slot][H][D][Dv]
//   head_norm_gate    o / rms(o) over each head's Dv * w * silu(gate) (or sigmoid(gate), or no gate)
#include "elem.h"

namespace lwc {
namespace {

template <typename IT, typename OT, int MODE>
__global__ void conv_hist_kernel(const IT* __restrict__ x, int ldx, const float* __restrict__ w, int ws_c, int ws_j,
                                 float* __restrict__ hist, long long slot_stride, const int* __restrict__ row_item,
                                 const int* __restrict__ cu, const int* __restrict__ item_slot,
                                 const int* __restrict__ positions, OT* __restrict__ out, int ldo, OT* __restrict__ out2,
                                 int ldo2, int C, int taps, int fuse) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int i = row_item[t];
  const int r = t - cu[i], p = positions[t];
  float* h = hist + (long long)item_slot[i] * slot_stride;
  const float cur = Elem<IT>::ld(x + (size_t)t * ldx + c);
  float acc = w[(size_t)c * ws_c + (size_t)(taps - 1) * ws_j] * cur;
  if (fuse) {  // every item is ONE row: this thread alone reads and rewrites its channel of the slot's history
    for (int s = taps - 1; s >= 1; --s) {
      const int e = taps - 1 - s;  // the entry that holds the input s rows back (meaningless before the start)
      const float v = h[(size_t)e * C + c];
      if (e >= 1) h[(size_t)(e - 1) * C + c] = v;
      acc += w[(size_t)c * ws_c + (size_t)(taps - 1 - s) * ws_j] * (s <= p ? v : 0.f);
    }
    if (taps > 1) h[(size_t)(taps - 2) * C + c] = cur;
  }
  for (int s = 1; s < taps && !fuse; ++s) {
    float v = 0.f;
    if (s <= r) v = Elem<IT>::ld(x + (size_t)(t - s) * ldx + c);
    else if (s <= p) v = h[(size_t)(taps - 1 - (s - r)) * C + c];
    acc += w[(size_t)c * ws_c + (size_t)(taps - 1 - s) * ws_j] * v;
  }
  if (MODE == 0) {
    Elem<OT>::st(out + (size_t)t * ldo + c, cur + acc);
    if (out2) Elem<OT>::st(out2 + (size_t)t * ldo2 + c, cur);
  } else {
    Elem<OT>::st(out + (size_t)t * ldo + c, MODE == 1 ? silu_f(acc) : acc);
  }
}

// Four channels per thread: weights stored tap-major (w[j][c]), every row base a multiple of four channels.
template <typename IT, typename OT, int MODE>
__global__ void conv_hist_vec_kernel(const IT* __restrict__ x, int ldx, const float* __restrict__ w,
                                     float* __restrict__ hist, long long slot_stride,
                                     const int* __restrict__ row_item, const int* __restrict__ cu,
                                     const int* __restrict__ item_slot, const int* __restrict__ positions,
                                     OT* __restrict__ out, int ldo, OT* __restrict__ out2, int ldo2, int C, int taps,
                                     int fuse) {
  const int t = blockIdx.y;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  const int i = row_item[t];
  const int r = t - cu[i], p = positions[t];
  float* h = hist + (long long)item_slot[i] * slot_stride;
  const float4v cur = Vec4<IT>::ld(x + (size_t)t * ldx + c);
  float4v acc = Vec4<float>::ld(w + (size_t)(taps - 1) * C + c) * cur;
  if (fuse) {  // every item is ONE row: this thread alone reads and rewrites its channels of the slot's history
    for (int s = taps - 1; s >= 1; --s) {
      const int e = taps - 1 - s;
      const float4v v = Vec4<float>::ld(h + (size_t)e * C + c);
      if (e >= 1) Vec4<float>::st(h + (size_t)(e - 1) * C + c, v);
      if (s <= p) acc += Vec4<float>::ld(w + (size_t)(taps - 1 - s) * C + c) * v;
    }
    if (taps > 1) Vec4<float>::st(h + (size_t)(taps - 2) * C + c, cur);
  }
  for (int s = 1; s < taps && !fuse; ++s) {
    float4v v = float4v{0.f, 0.f, 0.f, 0.f};
    if (s <= r) v = Vec4<IT>::ld(x + (size_t)(t - s) * ldx + c);
    else if (s <= p) v = Vec4<float>::ld(h + (size_t)(taps - 1 - (s - r)) * C + c);
    acc += Vec4<float>::ld(w + (size_t)(taps - 1 - s) * C + c) * v;
  }
  if (MODE == 0) {
    Vec4<OT>::st(out + (size_t)t * ldo + c, cur + acc);
    if (out2) Vec4<OT>::st(out2 + (size_t)t * ldo2 + c, cur);
  } else {
    Vec4<OT>::st(out + (size_t)t * ldo + c, MODE == 1 ? float4v{silu_f(acc[0]), silu_f(acc[1]), silu_f(acc[2]), silu_f(acc[3])} : acc);
  }
}

// Four channels x R consecutive rows per thread (taps <= 8): a row's earlier inputs stay in registers from the rows
// before it, so x is read about once instead of `taps` times and the weights once per thread.
template <typename IT, typename OT, int MODE, int R>
__global__ void conv_hist_tile_kernel(const IT* __restrict__ x, int ldx, const float* __restrict__ w,
                                      const float* __restrict__ hist, long long slot_stride,
                                      const int* __restrict__ row_item, const int* __restrict__ cu,
                                      const int* __restrict__ item_slot, const int* __restrict__ positions,
                                      OT* __restrict__ out, int ldo, OT* __restrict__ out2, int ldo2, int C, int taps,
                                      int T) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  const int t0 = blockIdx.y * R;
  const float4v zero = float4v{0.f, 0.f, 0.f, 0.f};
  float4v wv[8], prev[7];  // wv[s]: the weight of the input s rows back; prev[s - 1]: that input
#pragma unroll
  for (int s = 0; s < 8; ++s) wv[s] = s < taps ? Vec4<float>::ld(w + (size_t)(taps - 1 - s) * C + c) : zero;
#pragma unroll
  for (int s = 1; s < 8; ++s) prev[s - 1] = (s < taps && t0 - s >= 0) ? Vec4<IT>::ld(x + (size_t)(t0 - s) * ldx + c) : zero;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int t = t0 + j;
    if (t >= T) break;
    const int i = row_item[t];
    const int r = t - cu[i], p = positions[t];
    const float* h = hist + (long long)item_slot[i] * slot_stride;
    const float4v cur = Vec4<IT>::ld(x + (size_t)t * ldx + c);
    float4v acc = wv[0] * cur;
#pragma unroll
    for (int s = 1; s < 8; ++s) {
      if (s < taps) {
        float4v v = zero;
        if (s <= r) v = prev[s - 1];
        else if (s <= p) v = Vec4<float>::ld(h + (size_t)(taps - 1 - (s - r)) * C + c);
        acc += wv[s] * v;
      }
    }
    if (MODE == 0) {
      Vec4<OT>::st(out + (size_t)t * ldo + c, cur + acc);
      if (out2) Vec4<OT>::st(out2 + (size_t)t * ldo2 + c, cur);
    } else {
      Vec4<OT>::st(out + (size_t)t * ldo + c, MODE == 1 ? float4v{silu_f(acc[0]), silu_f(acc[1]), silu_f(acc[2]), silu_f(acc[3])} : acc);
    }
#pragma unroll
    for (int s = 6; s >= 1; --s) prev[s] = prev[s - 1];
    prev[0] = cur;
  }
}

constexpr int kMaxTaps = 16;

template <typename IT>
__global__ void conv_hist_update_kernel(const IT* __restrict__ x, int ldx, float* __restrict__ hist, long long slot_stride,
                                        const int* __restrict__ cu, const int* __restrict__ item_slot, int C, int taps) {
  const int i = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int K = taps - 1, r0 = cu[i], n = cu[i + 1] - r0;
  float* h = hist + (long long)item_slot[i] * slot_stride;
  float old[kMaxTaps];
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) old[j] = j < K ? h[(size_t)j * C + c] : 0.f;
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) {
    if (j < K) {
      const int idx = n - K + j;
      float v;
      if (idx >= 0) {
        v = Elem<IT>::ld(x + (size_t)(r0 + idx) * ldx + c);
      } else {
        v = 0.f;
#pragma unroll
        for (int m = 0; m < kMaxTaps; ++m) v = (m == j + n) ? old[m] : v;
      }
      h[(size_t)j * C + c] = v;
    }
  }
}

// Before the recurrence, per row and in parallel over rows: q and k (fp32 rows [q (G*D) | k (G*D) | v (H*Dv)]) made
// unit vectors per head IN PLACE (q also times D^-1/2), and bg[t] = [beta_h | decay_h | (q . k)_g] with beta and the
// decay from the projection columns ba[:, b_off + h], ba[:, a_off + h].
template <typename AT>
__global__ void delta_prep_kernel(float* __restrict__ qkv, int ldq, const AT* __restrict__ ba, int ldb, int b_off,
                                  int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                  float* __restrict__ bg, int H, int G, int D) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float qscale = 1.0f / sqrtf((float)D);
  for (int v = wv; v < 2 * G; v += nw) {  // q heads, then k heads
    float* x = qkv + (size_t)t * ldq + (size_t)v * D;
    float s = 0.f;
    for (int i = lane; i < D; i += 64) s += x[i] * x[i];
    const float r = (v < G ? qscale : 1.0f) / sqrtf(wave_sum(s) + 1e-6f);
    for (int i = lane; i < D; i += 64) x[i] *= r;
  }
  const int nb = 2 * H + G;  // bg row: beta_h | decay_h | (q . k)_g
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    bg[(size_t)t * nb + h] = sigmoid_f(Elem<AT>::ld(ba + (size_t)t * ldb + b_off + h));
    bg[(size_t)t * nb + H + h] = expf(-expf(A_log[h]) * softplus_f(Elem<AT>::ld(ba + (size_t)t * ldb + a_off + h) + dt_bias[h]));
  }
  __syncthreads();  // the normalised q and k of this row are written
  for (int g = wv; g < G; g += nw) {
    const float* q = qkv + (size_t)t * ldq + (size_t)g * D;
    const float* k = q + (size_t)G * D;
    float s = 0.f;
    for (int i = lane; i < D; i += 64) s += q[i] * k[i];
    s = wave_sum(s);
    if (lane == 0) bg[(size_t)t * nb + 2 * H + g] = s;
  }
}

// The recurrence: a workgroup of NW waves per (item, head, 16 NW value columns), one wave per 16 columns; lane =
// 16 r + c holds rows [r DPL, (r + 1) DPL) of state column c, so a token costs D / 4 multiply-adds per lane for each
// of the two dot products and the two updates, and the partial dot products meet through two lane swaps.  A
// token's k and q (shared by all columns of the head) are staged through LDS, double-buffered: the next token's
// operands are in flight while the current one is computed, one barrier per token.
template <int DPL, int NW>
__global__ void __launch_bounds__(64 * NW) delta_rule_kernel(const float* __restrict__ qkv, int ldq,
                                                              const float* __restrict__ bg, float* __restrict__ state,
                                                              long long slot_stride, const int* __restrict__ cu,
                                                              const int* __restrict__ item_slot,
                                                              const int* __restrict__ positions, float* __restrict__ out,
                                                              int ldo, int H, int G, int D, int Dv, int groups) {
  constexpr int QLD = DPL + 4;               // a quarter's row in LDS, padded against bank conflicts
  constexpr int PER = (8 * DPL + 64 * NW - 1) / (64 * NW);  // staged floats per thread (k and q: 2 * 4 DPL)
  __shared__ __attribute__((aligned(16))) float kq_s[2][2][4 * QLD];  // [buffer][k | q][quarter rows]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, c = lane & 15, r = lane >> 4;
  const int item = blockIdx.y, h = blockIdx.x / groups, grp = blockIdx.x - h * groups;
  const int col = (grp * NW + wv) * 16 + c;
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
  const int nq = G * D;
  // a token's operands in registers on their way to LDS: its chunk of k and q, its value, beta, decay and q . k
  struct Stage {
    float kq[PER], v, beta, g, qk;
  };
  const int nb = 2 * H + G;
  auto fetch = [&](int row, Stage& st) {
    const float* qr = qkv + (size_t)row * ldq + kvh * D;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 64 * NW * u;       // e < 4 DPL: k row e; else q row e - 4 DPL
      const int which = e >= 4 * DPL, i = e - which * 4 * DPL;
      st.kq[u] = (e < 8 * DPL && i < D) ? qr[(which ? 0 : nq) + i] : 0.f;
    }
    st.v = live ? qkv[(size_t)row * ldq + 2 * nq + h * Dv + col] : 0.f;
    st.beta = bg[(size_t)row * nb + h];
    st.g = bg[(size_t)row * nb + H + h];
    st.qk = bg[(size_t)row * nb + 2 * H + kvh];
  };
  auto stash = [&](int buf, const Stage& st) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 64 * NW * u;
      const int which = e >= 4 * DPL, i = e - which * 4 * DPL;
      if (e < 8 * DPL) kq_s[buf][which][(i / DPL) * QLD + i % DPL] = st.kq[u];
    }
  };
  // Two register stages alternate, so a token's loads are issued two tokens before they are needed (one token's
  // arithmetic is shorter than a trip to memory).
  Stage A, B;
  fetch(r0, A);
  stash(0, A);
  float v = A.v, beta = A.beta, g = A.g, qk = A.qk;
  if (r0 + 1 < r1) fetch(r0 + 1, A);
  if (r0 + 2 < r1) fetch(r0 + 2, B);
  __syncthreads();
  // one token out of LDS buffer `cur`; `next` holds the following token's operands and is refilled three ahead
  auto step = [&](int row, int cur, Stage& next) {
    const float4v* ks = reinterpret_cast<const float4v*>(&kq_s[cur][0][r * QLD]);
    const float4v* qs = reinterpret_cast<const float4v*>(&kq_s[cur][1][r * QLD]);
    // With S the state BEFORE this token: S^T k and S^T q in one pass (independent partial sums), then
    //   u = beta (v - g S^T k),   o = (g S + k u^T)^T q = g S^T q + (k . q) u,   S <- g S + k u^T
    float kk[DPL];
    float4v dk = float4v{0.f, 0.f, 0.f, 0.f}, dq = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < DPL / 4; ++j) {
      const float4v k4 = ks[j], q4 = qs[j];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        kk[4 * j + e] = k4[e];
        dk[e] += S[4 * j + e] * k4[e];
        dq[e] += S[4 * j + e] * q4[e];
      }
    }
    const float sk = row_sum4((dk[0] + dk[1]) + (dk[2] + dk[3]));
    const float sq = row_sum4((dq[0] + dq[1]) + (dq[2] + dq[3]));
    const float u = beta * (v - g * sk);
    if (live && r == 0) out[(size_t)row * ldo + h * Dv + col] = g * sq + qk * u;
#pragma unroll
    for (int j = 0; j < DPL; ++j) S[j] = kk[j] * u + g * S[j];
    if (row + 1 < r1) {
      stash(cur ^ 1, next);
      v = next.v, beta = next.beta, g = next.g, qk = next.qk;
      if (row + 3 < r1) fetch(row + 3, next);
    }
    __syncthreads();
  };
  for (int row = r0; row < r1; row += 2) {
    step(row, 0, A);
    if (row + 1 < r1) step(row + 1, 1, B);
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < DPL; ++j)
      if (i0 + j < D) Sg[(size_t)j * Dv] = S[j];
  }
}

// GATE 0: none, 1: silu(gate), 2: sigmoid(gate)
template <typename AT, int GATE>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, int ldi, const AT* __restrict__ gate, int ldg,
                                      const float* __restrict__ w, AT* __restrict__ out, int ldo, int H, int Dv,
                                      float eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int h = wv; h < H; h += nw) {
    const float* oh = o + (size_t)t * ldi + h * Dv;
    float s = 0.f;
    for (int i = lane; i < Dv; i += 64) s += oh[i] * oh[i];
    const float rstd = 1.0f / sqrtf(wave_sum(s) / (float)Dv + eps);
    for (int i = lane; i < Dv; i += 64) {
      float y = oh[i] * rstd * (w ? w[i] : 1.0f);
      if (GATE) {
        const float z = Elem<AT>::ld(gate + (size_t)t * ldg + h * Dv + i);
        y *= GATE == 1 ? silu_f(z) : sigmoid_f(z);
      }
      Elem<AT>::st(out + (size_t)t * ldo + h * Dv + i, y);
    }
  }
}

// Dv a multiple of four, aligned bases: 16-byte reads of o, four gate values per lane
template <typename AT, int GATE>
__global__ void head_norm_gate_vec_kernel(const float* __restrict__ o, int ldi, const AT* __restrict__ gate, int ldg,
                                          const float* __restrict__ w, AT* __restrict__ out, int ldo, int H, int Dv,
                                          float eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int h = wv; h < H; h += nw) {
    const float* oh = o + (size_t)t * ldi + h * Dv;
    float s = 0.f;
    for (int i = lane * 4; i < Dv; i += 256) {
      const float4v v = Vec4<float>::ld(oh + i);
      s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    const float rstd = 1.0f / sqrtf(wave_sum(s) / (float)Dv + eps);
    for (int i = lane * 4; i < Dv; i += 256) {
      float4v y = Vec4<float>::ld(oh + i) * rstd;
      if (w) y *= Vec4<float>::ld(w + i);
      if (GATE) {
        const float4v z = Vec4<AT>::ld(gate + (size_t)t * ldg + h * Dv + i);
        y *= GATE == 1 ? float4v{silu_f(z[0]), silu_f(z[1]), silu_f(z[2]), silu_f(z[3])}
                       : float4v{sigmoid_f(z[0]), sigmoid_f(z[1]), sigmoid_f(z[2]), sigmoid_f(z[3])};
      }
      Vec4<AT>::st(out + (size_t)t * ldo + h * Dv + i, y);
    }
  }
}

// Dv / 4 a power of two <= 64: LPH = Dv / 4 lanes per head, 64 / LPH heads per wave at once, every lane busy
template <typename AT, int GATE>
__global__ void head_norm_gate_sub_kernel(const float* __restrict__ o, int ldi, const AT* __restrict__ gate, int ldg,
                                          const float* __restrict__ w, AT* __restrict__ out, int ldo, int H, int Dv,
                                          float eps, int LPH) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int hpw = 64 / LPH, sub = lane / LPH, i = (lane - sub * LPH) * 4;
  for (int h0 = wv * hpw; h0 < H; h0 += nw * hpw) {
    const int h = h0 + sub;
    const bool ok = h < H;
    const float* oh = o + (size_t)t * ldi + (ok ? h : 0) * Dv;
    const float4v v = Vec4<float>::ld(oh + i);
    float s = v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    for (int m = LPH >> 1; m > 0; m >>= 1) s += __shfl_xor(s, m, 64);
    const float rstd = 1.0f / sqrtf(s / (float)Dv + eps);
    float4v y = v * rstd;
    if (w) y *= Vec4<float>::ld(w + i);
    if (ok) {
      if (GATE) {
        const float4v z = Vec4<AT>::ld(gate + (size_t)t * ldg + h * Dv + i);
        y *= GATE == 1 ? float4v{silu_f(z[0]), silu_f(z[1]), silu_f(z[2]), silu_f(z[3])}
                       : float4v{sigmoid_f(z[0]), sigmoid_f(z[1]), sigmoid_f(z[2]), sigmoid_f(z[3])};
      }
      Vec4<AT>::st(out + (size_t)t * ldo + h * Dv + i, y);
    }
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

// io: bit 0 = input fp32 (else bf16), bit 1 = output fp32 (else bf16)
// w: element (c, j) at w[c * ws_c + j * ws_j]
// fuse != 0: every item is one row (T == items) and the slot's history is advanced by the same kernel
extern "C" int r32_conv_hist(const void* x, int ldx, const float* w, int ws_c, int ws_j, float* hist,
                             long long slot_stride, const int* row_item, const int* cu, const int* item_slot,
                             const int* positions, void* out, int ldo, void* out2, int ldo2, int T, int C, int taps,
                             int mode, int io, int fuse, hipStream_t s) {
  if (T <= 0 || C <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps) return -1;
  const int ib = (io & 1) ? 16 : 8, ob = (io & 2) ? 16 : 8;
  const bool vec = ws_c == 1 && (taps == 1 || ws_j == C) && C % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && ldo2 % 4 == 0 &&
                   slot_stride % 4 == 0 && aligned_to(x, ib) && aligned_to(out, ob) && aligned_to(out2, ob) &&
                   aligned_to(w, 16) && aligned_to(hist, 16);
  const int threads = vec && C / 4 <= 64 ? 64 : (vec && C / 4 <= 128 ? 128 : 256);
  dim3 grid(vec ? (C / 4 + threads - 1) / threads : (C + 255) / 256, T);
  constexpr int kRows = 8;
  const bool tile = vec && !fuse && taps <= 8 && T >= 8 * kRows;
  dim3 tgrid(grid.x, (T + kRows - 1) / kRows);
#define LWC_CONV(IT, OT, M)                                                                                            \
  if (tile)                                                                                                            \
    conv_hist_tile_kernel<IT, OT, M, kRows><<<tgrid, threads, 0, s>>>((const IT*)x, ldx, w, hist, slot_stride,        \
                                                                       row_item, cu, item_slot, positions, (OT*)out,  \
                                                                       ldo, (OT*)out2, ldo2, C, taps, T);             \
  else if (vec)                                                                                                        \
    conv_hist_vec_kernel<IT, OT, M><<<grid, threads, 0, s>>>((const IT*)x, ldx, w, hist, slot_stride, row_item, cu,   \
                                                             item_slot, positions, (OT*)out, ldo, (OT*)out2, ldo2, C, \
                                                             taps, fuse);                                              \
  else                                                                                                                 \
    conv_hist_kernel<IT, OT, M><<<grid, threads, 0, s>>>((const IT*)x, ldx, w, ws_c, ws_j, hist, slot_stride,         \
                                                         row_item, cu, item_slot, positions, (OT*)out, ldo,            \
                                                         (OT*)out2, ldo2, C, taps, fuse)
  if (mode == 0) {
    if (io == 3) {
      LWC_CONV(float, float, 0);
    } else if (io == 1) {
      LWC_CONV(float, bf16_t, 0);
    } else if (io == 0) {
      LWC_CONV(bf16_t, bf16_t, 0);
    } else {
      return -1;
    }
  } else if (mode == 1) {
    if (io == 3) {
      LWC_CONV(float, float, 1);
    } else if (io == 2) {
      LWC_CONV(bf16_t, float, 1);
    } else if (io == 0) {
      LWC_CONV(bf16_t, bf16_t, 1);
    } else {
      return -1;
    }
  } else if (mode == 2) {
    if (io == 3) {
      LWC_CONV(float, float, 2);
    } else if (io == 2) {
      LWC_CONV(bf16_t, float, 2);
    } else if (io == 0) {
      LWC_CONV(bf16_t, bf16_t, 2);
    } else {
      return -1;
    }
  } else {
    return -1;
  }
#undef LWC_CONV
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_conv_hist_update(const void* x, int ldx, float* hist, long long slot_stride, const int* cu,
                                    const int* item_slot, int items, int C, int taps, int in_f32, hipStream_t s) {
  if (items <= 0 || C <= 0 || taps <= 1) return 0;
  if (taps > kMaxTaps) return -1;
  dim3 grid((C + 255) / 256, items);
  if (in_f32) conv_hist_update_kernel<float><<<grid, 256, 0, s>>>((const float*)x, ldx, hist, slot_stride, cu, item_slot, C, taps);
  else conv_hist_update_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, ldx, hist, slot_stride, cu, item_slot, C, taps);
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_delta_rule_max_dim() { return 256; }

// qkv is normalised in place (q, k columns); bg fp32 [T, 2 H + G] scratch for beta, the decays and q . k
extern "C" int r32_delta_rule(float* qkv, int ldq, const void* ba, int ldb, int b_off, int a_off, const float* A_log,
                              const float* dt_bias, float* bg, float* state, long long slot_stride, const int* cu,
                              const int* item_slot, const int* positions, float* out, int ldo, int T, int items, int H,
                              int G, int D, int Dv, int f32, hipStream_t s) {
  if (items <= 0 || T <= 0) return 0;
  if (D < 1 || D > 256 || H % G != 0) return -1;
  if (f32) delta_prep_kernel<float><<<T, 256, 0, s>>>(qkv, ldq, (const float*)ba, ldb, b_off, a_off, A_log, dt_bias, bg, H, G, D);
  else delta_prep_kernel<bf16_t><<<T, 256, 0, s>>>(qkv, ldq, (const bf16_t*)ba, ldb, b_off, a_off, A_log, dt_bias, bg, H, G, D);
  const int tiles = (Dv + 15) / 16;
#define LWC_DELTA(DPL, NW)                                                                                          \
  delta_rule_kernel<DPL, NW><<<dim3(H * ((tiles + NW - 1) / NW), items), 64 * NW, 0, s>>>(                         \
      qkv, ldq, bg, state, slot_stride, cu, item_slot, positions, out, ldo, H, G, D, Dv, (tiles + NW - 1) / NW)
#define LWC_DELTA_NW(DPL)      \
  if (tiles >= 4) {            \
    LWC_DELTA(DPL, 4);         \
  } else if (tiles >= 2) {     \
    LWC_DELTA(DPL, 2);         \
  } else {                     \
    LWC_DELTA(DPL, 1);         \
  }
  if (D <= 32) {
    LWC_DELTA_NW(8)
  } else if (D <= 64) {
    LWC_DELTA_NW(16)
  } else if (D <= 128) {
    LWC_DELTA_NW(32)
  } else {
    LWC_DELTA_NW(64)
  }
#undef LWC_DELTA_NW
#undef LWC_DELTA
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_head_norm_gate(const float* o, int ldi, const void* gate, int ldg, const float* w, void* out, int ldo,
                                  int T, int H, int Dv, float eps, int gate_mode, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  const int threads = H >= 4 ? 256 : 64 * H;
  const int ab = f32 ? 16 : 8;
  const bool vec = Dv % 4 == 0 && ldi % 4 == 0 && ldg % 4 == 0 && ldo % 4 == 0 && aligned_to(o, 16) && aligned_to(w, 16) &&
                   aligned_to(gate, ab) && aligned_to(out, ab);
  const int lph = Dv / 4;
  const bool sub = vec && lph >= 1 && lph <= 64 && (lph & (lph - 1)) == 0;
#define LWC_HNG(AT, GM)                                                                                                  \
  if (sub)                                                                                                               \
    head_norm_gate_sub_kernel<AT, GM><<<T, threads, 0, s>>>(o, ldi, (const AT*)gate, ldg, w, (AT*)out, ldo, H, Dv, eps,  \
                                                            lph);                                                        \
  else if (vec)                                                                                                          \
    head_norm_gate_vec_kernel<AT, GM><<<T, threads, 0, s>>>(o, ldi, (const AT*)gate, ldg, w, (AT*)out, ldo, H, Dv, eps); \
  else                                                                                                                   \
    head_norm_gate_kernel<AT, GM><<<T, threads, 0, s>>>(o, ldi, (const AT*)gate, ldg, w, (AT*)out, ldo, H, Dv, eps)
  if (f32) {
    if (gate_mode == 0) {
      LWC_HNG(float, 0);
    } else if (gate_mode == 1) {
      LWC_HNG(float, 1);
    } else {
      LWC_HNG(float, 2);
    }
  } else {
    if (gate_mode == 0) {
      LWC_HNG(bf16_t, 0);
    } else if (gate_mode == 1) {
      LWC_HNG(bf16_t, 1);
    } else {
      LWC_HNG(bf16_t, 2);
    }
  }
#undef LWC_HNG
  LWC_CHECK_LAUNCH();
  return 0;
}

// Retention: linear attention with a fixed decay per head and no softmax (gfx950, wave64).
//
//   S_t = a_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t          S fp32 [D, Dv] per head and sequence
// q and k are rotated by position on their first `rd` entries ("rotate half": entry i pairs with i + rd / 2, angle
// p * f_i as an fp32 product), k is then multiplied by D^-1/2.  Everything that enters the recurrence is fp32.
//
//   retention_prep   q, k of a step's rows (activation type) -> rotated, scaled fp32 rows [T, 2, H, D]
//   retention        the recurrence over a step's items (rows of one sequence at consecutive positions + the
//                    sequence's state slot; a decode row is an item of one row).  One workgroup of NW waves per (item,
//                    head, 16 NW value columns): a lane keeps a quarter of one state column in registers (lane =
//                    quarter * 16 + column), the q / k / v of TT tokens are staged through LDS at once (one barrier
//                    pair per TT tokens), the four partial dots of a column meet by two half-wave swaps.  The state is
//                    read from the slot unless the item starts at position 0, and written back at the end.
#include "elem.h"

namespace lwc {
namespace {

template <typename AT>
__global__ void __launch_bounds__(256)
retention_prep_kernel(const AT* __restrict__ proj, int ldp, int k_off, const float* __restrict__ freq, float mult,
                      const int* __restrict__ positions, float* __restrict__ qk, int H, int D, int rd, float k_scale) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const AT* pr = proj + (size_t)t * ldp;
  float* o = qk + (size_t)t * 2 * H * D;
  const int half = rd / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {  // one angle serves every head, q and k
    float sn, cs;
    sincosf(p * freq[i], &sn, &cs);
    sn *= mult, cs *= mult;
    for (int h = 0; h < H; ++h) {
      const int c = h * D + i;
      const float qu = Elem<AT>::ld(pr + c), qv = Elem<AT>::ld(pr + c + half);
      const float ku = Elem<AT>::ld(pr + k_off + c), kv = Elem<AT>::ld(pr + k_off + c + half);
      o[c] = qu * cs - qv * sn;
      o[c + half] = qv * cs + qu * sn;
      o[H * D + c] = (ku * cs - kv * sn) * k_scale;
      o[H * D + c + half] = (kv * cs + ku * sn) * k_scale;
    }
  }
  const int rest = D - rd;
  for (int e = threadIdx.x; e < H * rest; e += blockDim.x) {
    const int h = e / rest, c = h * D + rd + (e - h * rest);
    o[c] = Elem<AT>::ld(pr + c);
    o[H * D + c] = Elem<AT>::ld(pr + k_off + c) * k_scale;
  }
}

constexpr int kTT = 16;  // tokens staged at once

template <typename AT, int DPL, int NW>
__global__ void __launch_bounds__(64 * NW)
retention_kernel(const float* __restrict__ qk, const AT* __restrict__ v, int ldv, const float* __restrict__ decay,
                 float* __restrict__ state, long long slot_stride, const int* __restrict__ cu,
                 const int* __restrict__ item_slot, const int* __restrict__ positions, float* __restrict__ out, int ldo,
                 int H, int D, int Dv, int col_tiles) {
  constexpr int QLD = DPL + 4;   // a quarter's stride in LDS: the four quarters start in different banks
  constexpr int VT = 16 * NW;    // value columns of a workgroup
  __shared__ __attribute__((aligned(16))) float q_s[kTT][4 * QLD];
  __shared__ __attribute__((aligned(16))) float k_s[kTT][4 * QLD];
  __shared__ float v_s[kTT][VT];
  const int item = blockIdx.y;
  const int h = blockIdx.x / col_tiles, col0 = (blockIdx.x % col_tiles) * VT;
  const int r0 = cu[item], r1 = cu[item + 1];
  if (r0 >= r1) return;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int r = lane >> 4, cl = wv * 16 + (lane & 15), col = col0 + cl;
  const bool live = col < Dv;
  const int i0 = r * DPL;
  const float a = decay[h];
  float* Sg = state + (long long)item_slot[item] * slot_stride + ((size_t)h * D + i0) * Dv + (live ? col : 0);
  float S[DPL];
  const bool fresh = positions[r0] == 0;
#pragma unroll
  for (int j = 0; j < DPL; ++j) S[j] = (!fresh && live && i0 + j < D) ? Sg[(size_t)j * Dv] : 0.f;
  for (int t0 = r0; t0 < r1; t0 += kTT) {
    const int nt = min(kTT, r1 - t0);
    __syncthreads();  // the previous tile has been read
    for (int e = tid; e < nt * 4 * DPL; e += 64 * NW) {
      const int tt = e / (4 * DPL), i = e - tt * (4 * DPL);
      const float* row = qk + (size_t)(t0 + tt) * 2 * H * D + (size_t)h * D;
      const int at = (i / DPL) * QLD + (i % DPL);
      q_s[tt][at] = i < D ? row[i] : 0.f;
      k_s[tt][at] = i < D ? row[H * D + i] : 0.f;
    }
    for (int e = tid; e < nt * VT; e += 64 * NW) {
      const int tt = e / VT, c = e - tt * VT;
      v_s[tt][c] = col0 + c < Dv ? Elem<AT>::ld(v + (size_t)(t0 + tt) * ldv + (size_t)h * Dv + col0 + c) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float4v* ks = reinterpret_cast<const float4v*>(&k_s[tt][r * QLD]);
      const float4v* qs = reinterpret_cast<const float4v*>(&q_s[tt][r * QLD]);
      const float vv = v_s[tt][cl];
      float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < DPL / 4; ++j) {
        const float4v k4 = ks[j], q4 = qs[j];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[4 * j + e] = a * S[4 * j + e] + k4[e] * vv;
          acc[e] += S[4 * j + e] * q4[e];
        }
      }
      const float o = row_sum4((acc[0] + acc[1]) + (acc[2] + acc[3]));
      if (live && r == 0) out[(size_t)(t0 + tt) * ldo + (size_t)h * Dv + col] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < DPL; ++j)
      if (i0 + j < D) Sg[(size_t)j * Dv] = S[j];
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_retention_max_dim() { return 256; }

extern "C" int r32_retention_prep(const void* proj, int ldp, int k_off, const float* freq, float mult, const int* positions,
                                  float* qk, int T, int H, int D, int rd, float k_scale, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (rd % 2 != 0 || rd > D || rd < 0) return -1;
  if (f32) retention_prep_kernel<float><<<T, 256, 0, s>>>((const float*)proj, ldp, k_off, freq, mult, positions, qk, H, D, rd, k_scale);
  else retention_prep_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)proj, ldp, k_off, freq, mult, positions, qk, H, D, rd, k_scale);
  LWC_CHECK_LAUNCH();
  return 0;
}

// qk fp32 [T, 2, H, D] from retention_prep; v rows of the activation type (leading dimension ldv), head h at columns
// h Dv ..; state fp32 [slots, H, D, Dv]; out fp32 rows (leading dimension ldo)
extern "C" int r32_retention(const float* qk, const void* v, int ldv, const float* decay, float* state, long long slot_stride,
                             const int* cu, const int* item_slot, const int* positions, float* out, int ldo, int items,
                             int H, int D, int Dv, int f32, hipStream_t s) {
  if (items <= 0) return 0;
  if (D < 1 || D > 256 || Dv < 1) return -1;
  const int tiles = (Dv + 15) / 16;
#define LWC_RET2(AT, DPL, NW)                                                                                             \
  retention_kernel<AT, DPL, NW><<<dim3(H * ((tiles + NW - 1) / NW), items), 64 * NW, 0, s>>>(                            \
      qk, (const AT*)v, ldv, decay, state, slot_stride, cu, item_slot, positions, out, ldo, H, D, Dv, (tiles + NW - 1) / NW)
#define LWC_RET(DPL, NW)       \
  if (f32) {                   \
    LWC_RET2(float, DPL, NW);  \
  } else {                     \
    LWC_RET2(bf16_t, DPL, NW); \
  }
#define LWC_RET_NW(DPL)    \
  if (tiles >= 4) {        \
    LWC_RET(DPL, 4)        \
  } else if (tiles >= 2) { \
    LWC_RET(DPL, 2)        \
  } else {                 \
    LWC_RET(DPL, 1)        \
  }
  if (D <= 32) {
    LWC_RET_NW(8)
  } else if (D <= 64) {
    LWC_RET_NW(16)
  } else if (D <= 128) {
    LWC_RET_NW(32)
  } else {
    LWC_RET_NW(64)
  }
#undef LWC_RET_NW
#undef LWC_RET
#undef LWC_RET2
  LWC_CHECK_LAUNCH();
  return 0;
}

// Decode rows of the sliding-window attention (see wattn.hip for the scores, the cache layout and the portion kernel).
#pragma once
#include "../common.h"

using namespace lwc;

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

LWC_DEVICE float4v mfma16(const short8& a, const short8& b, const float4v& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// ---------------------------------------------------------------------------------------------------------
// window_attn_decode_kernel: one new token per sequence on the matrix cores (bf16 cache), split over the keys.
//
// One wave per (sequence b, key/value head g, head chunk, key split).  The N = 16 columns of the MFMA are the
// (up to 16) query heads that share head g, so K and V are read ONCE for all of them, straight from the paged
// cache into the operands — no LDS: a K row's 16 bytes are an A operand as they lie, the interleaved V word is a
// B operand as it lies.  Same arithmetic as the portion kernel (hi + lo halves of q and of the weights, bias
// table, fp32 online softmax).  Each split leaves an unnormalised partial (o, m, l); the reduce kernel merges
// them (splits == 1: still through the reduce, which then only normalises).
struct WAttnDecodeParams {
  const float* q;          // [B, H*D]
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  long long kb_stride, vb_stride;
  int block_size, bs_shift;  // block_size = 1 << bs_shift (the matrix-core kernels take power-of-two pages)
  const int* positions;    // [B]: the new token's position (its key is already in the cache)
  const int* block_tables;
  int bt_width;
  const float* bias;       // [H, window], or null: no distance bias
  int window;
  int chunk;               // > 0: the row sees only keys of its own chunk, j >= i - i % chunk (besides the window)
  float* part_o;           // [B, H, S, Dv]
  float* part_ml;          // [B, H, S, 2]
  int H, G, S, keys_per_split;  // keys_per_split: a multiple of 32
};

// NW waves per workgroup share one (sequence, head chunk, split).  With NW > 1 a tile's 32 key rows go through LDS
// once for all the waves (fetched into registers one tile ahead), and each wave owns NV / NW of the 16-column value
// tiles (wide value rows: the accumulators of one wave would leave no registers for loads in flight).  NW = 4: the
// waves also form the tile's scores together, each a quarter of the MFMAs (one key subtile times half of the row's
// 32-entry slices), and the partial scores meet in LDS.
// QLO = false: q enters as its bf16 rounding only (one MFMA per operand instead of two).
// VK = true (with NW > 1): the values ARE the first DV entries of the key rows (a cached latent that is key and value
// at once), so the value operands are gathered from the staged rows in LDS and the value pages are not read at all.
// NC > 1: NC head chunks (16 heads each) of one kv head share the workgroup and with it every staged key row (waves
// [c NW, (c + 1) NW) serve chunk c).
template <int ND, int NV, int NW = 1, bool QLO = true, bool VK = false, int NC = 1>
__global__ void __launch_bounds__(64 * NW * NC) window_attn_decode_kernel(const WAttnDecodeParams p) {
  constexpr int D = 32 * ND, DV = 16 * NV, NVW = NV / NW, NT = 64 * NW * NC;  // NT: threads of the workgroup
  static_assert(NV % NW == 0, "value tiles divide among the waves");
  const int b = blockIdx.x, split = blockIdx.z;
  const int H = p.H, G = p.G, Hg = H / G, chunks = (Hg + 15) / 16;
  // (one wave: the wave index is a compile-time zero, so the value tiles' offsets stay immediates)
  const int lane = NT > 64 ? (int)(threadIdx.x & 63) : (int)threadIdx.x, wv_all = NT > 64 ? (int)(threadIdx.x >> 6) : 0;
  const int wv = NC > 1 ? wv_all % NW : wv_all, cw = NC > 1 ? wv_all / NW : 0;
  const int cgroups = (chunks + NC - 1) / NC;  // workgroups per kv head
  const int g = blockIdx.y / cgroups, h0 = g * Hg + ((blockIdx.y % cgroups) * NC + cw) * 16;
  const int nh = min(16, g * Hg + Hg - h0);  // heads of this chunk (<= 0: a wave past the last chunk only helps staging)
  const int r16 = lane & 15, g4 = lane >> 4;
  const int i = p.positions[b];
  const int j_lo = max(max(0, i - p.window + 1), p.chunk > 0 ? i - i % p.chunk : 0);
  const int base = (j_lo / 32) * 32 + split * p.keys_per_split;  // this split's first key (a multiple of 32)
  const int last = min(i, base + p.keys_per_split - 1);
  const int* table = p.block_tables + (size_t)b * p.bt_width;
  const int BS = p.block_size, bsh = p.bs_shift;
  auto page_ix = [&](int j) { return j >> bsh; };
  auto page_off = [&](int j) { return j & (BS - 1); };
  // the split's pages, one per lane, fetched once: a key's page then comes from a lane exchange instead of a table
  // load that every K / V load would have to wait for (splits longer than 64 pages look the table up directly)
  const int pg_base = page_ix(base);
  const bool pages_in_lanes = page_ix(base + p.keys_per_split - 1) - pg_base < 64;
  int my_page = 0;
  if (pages_in_lanes && pg_base + lane <= page_ix(max(i, 0)) && base <= i) my_page = table[pg_base + lane];
  auto page_of = [&](int j) { return pages_in_lanes ? __shfl(my_page, page_ix(j) - pg_base, 64) : table[page_ix(j)]; };
  const bool h_valid = r16 < nh;
  const int h = h0 + (h_valid ? r16 : 0);

  // With NW = 4 staged waves the scores of a tile are formed ONCE per chunk: wave w multiplies key subtile (w & 1) with
  // half (w >> 1) of the row's 32-entry slices, the halves meet through LDS.  Such a wave keeps only its half of q.
  constexpr bool kSplitQK = NW == 4;
  static_assert(!kSplitQK || ND % 2 == 0, "the slices divide into two halves");
  constexpr int NDW = kSplitQK ? ND / 2 : ND;
  const int kd0 = kSplitQK ? (wv >> 1) * NDW : 0;
  short8 qhi[NDW], qlo[QLO ? NDW : 1];
#pragma unroll
  for (int kd = 0; kd < NDW; ++kd) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = 0.f;
      if (h_valid) x = p.q[((size_t)b * H + h) * D + (kd0 + kd) * 32 + 8 * g4 + e];
      const bf16_t hi = f2bf(x);
      qhi[kd][e] = (short)hi;
      if (QLO) qlo[kd][e] = (short)f2bf(x - bf2f(hi));
    }
  }
  float4v O[NVW];
#pragma unroll
  for (int n = 0; n < NVW; ++n) O[n] = float4v{0.f, 0.f, 0.f, 0.f};
  float m = -1e30f, l = 0.f;
  const float* bias_h = p.bias ? p.bias + (size_t)h * p.window : nullptr;  // no table: no distance bias

  constexpr bool kStage = NW > 1;
  constexpr int KLD = D + 8;                                       // LDS row stride: rows start in different banks
  constexpr int KCH = (32 * (D / 8) + NT - 1) / NT;                 // 16-byte words per thread and tile
  __shared__ __attribute__((aligned(16))) bf16_t K_s[kStage ? 32 * KLD : 8];
  __shared__ __attribute__((aligned(16))) float4v S_x[NW == 4 ? NC * NW * 64 : 1];  // partial scores of the waves
  uint4v kreg[kStage ? KCH : 1];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int c = min((int)threadIdx.x + NT * u, 32 * (D / 8) - 1);
      const int key = c / (D / 8), dc = c % (D / 8);
      const int j = min(t0 + key, i);  // (rows past the token are masked below: any valid row does)
      kreg[u] = *reinterpret_cast<const uint4v*>(p.k_cache + (long long)page_of(j) * p.kb_stride +
                                                 ((long long)page_off(j) * G + g) * D + dc * 8);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int c = (int)threadIdx.x + NT * u;
      if (c < 32 * (D / 8)) *reinterpret_cast<uint4v*>(&K_s[(c / (D / 8)) * KLD + (c % (D / 8)) * 8]) = kreg[u];
    }
  };
  if (kStage && base <= last) {
    fetch(base);
    stash();
    __syncthreads();
  }

  for (int t0 = base; t0 <= last; t0 += 32) {  // (base and last are the same for every wave of the workgroup)
    if (kStage && t0 + 32 <= last) fetch(t0 + 32);
    float4v sacc[2];
    if constexpr (kSplitQK) {
      float4v part = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kd = 0; kd < NDW; ++kd) {
        const short8 a = *reinterpret_cast<const short8*>(&K_s[((wv & 1) * 16 + r16) * KLD + (kd0 + kd) * 32 + 8 * g4]);
        part = mfma16(a, qhi[kd], part);
        if (QLO) part = mfma16(a, qlo[kd], part);
      }
      S_x[(cw * NW + wv) * 64 + lane] = part;
      __syncthreads();  // (the barriers at the tile's end keep the next tile's partials from overtaking these reads)
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
        sacc[sub] = S_x[(cw * NW + sub) * 64 + lane] + S_x[(cw * NW + sub + 2) * 64 + lane];
    } else {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      sacc[sub] = float4v{0.f, 0.f, 0.f, 0.f};
      if (kStage) {
#pragma unroll
        for (int kd = 0; kd < ND; ++kd) {
          const short8 a = *reinterpret_cast<const short8*>(&K_s[(sub * 16 + r16) * KLD + kd * 32 + 8 * g4]);
          sacc[sub] = mfma16(a, qhi[kd], sacc[sub]);
          if (QLO) sacc[sub] = mfma16(a, qlo[kd], sacc[sub]);
        }
      } else {
        const int j = min(t0 + sub * 16 + r16, i);  // (rows past the token are masked below: any valid row does)
        const bf16_t* kr = p.k_cache + (long long)page_of(j) * p.kb_stride + ((long long)page_off(j) * G + g) * D + 8 * g4;
#pragma unroll
        for (int kd = 0; kd < ND; ++kd) {
          const short8 a = *reinterpret_cast<const short8*>(kr + kd * 32);
          sacc[sub] = mfma16(a, qhi[kd], sacc[sub]);
          if (QLO) sacc[sub] = mfma16(a, qlo[kd], sacc[sub]);
        }
      }
    }
    }  // (scores without the split)
    float s[8];
    bool ok[8];
    float mx = -1e30f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = t0 + (e >> 2) * 16 + 4 * g4 + (e & 3);
      const int dist = i - j;
      ok[e] = h_valid && dist >= 0 && j >= j_lo && j <= last;
      s[e] = ok[e] ? sacc[e >> 2][e & 3] - (bias_h ? bias_h[dist] : 0.f) : -1e30f;
      mx = fmaxf(mx, s[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = expf(m - m_new);
    float pe[8], psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pe[e] = ok[e] ? expf(s[e] - m_new) : 0.f;
      psum += pe[e];
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
    short8 ph, pl;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const bf16_t hi = f2bf(pe[e]);
      ph[e] = (short)hi;
      pl[e] = (short)f2bf(pe[e] - bf2f(hi));
    }
    float ar[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) ar[r] = __shfl(alpha, 4 * g4 + r, 64);
    // the lane's two 4-key groups: keys t0 + 4 g4 .. and t0 + 16 + 4 g4 .. (groups past the token: any valid one,
    // their weights are 0)
    const int ja = min(t0 + 4 * g4, (i / 4) * 4), jb = min(t0 + 16 + 4 * g4, (i / 4) * 4);
    const bf16_t* va = p.v_cache + (long long)page_of(ja) * p.vb_stride + (long long)(page_off(ja) >> 2) * (4LL * G * DV) + 4LL * (g * DV + r16);
    const bf16_t* vb = p.v_cache + (long long)page_of(jb) * p.vb_stride + (long long)(page_off(jb) >> 2) * (4LL * G * DV) + 4LL * (g * DV + r16);
#pragma unroll
    for (int n = 0; n < NVW; ++n) {
#pragma unroll
      for (int r = 0; r < 4; ++r) O[n][r] *= ar[r];
      short8 bb;
      if (kStage && VK) {
        const bf16_t* col = &K_s[(4 * g4) * KLD + 16 * (wv * NVW + n) + r16];  // this lane's value column, key 4 g4
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          bb[e] = (short)col[e * KLD];
          bb[4 + e] = (short)col[(16 + e) * KLD];
        }
      } else {
        const short4v b0 = *reinterpret_cast<const short4v*>(va + 64 * (wv * NVW + n));
        const short4v b1 = *reinterpret_cast<const short4v*>(vb + 64 * (wv * NVW + n));
        bb = short8{b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
      }
      O[n] = mfma16(ph, bb, O[n]);
      O[n] = mfma16(pl, bb, O[n]);
    }
    if (kStage) {
      __syncthreads();  // every wave has read this tile's rows
      if (t0 + 32 <= last) stash();
      __syncthreads();
    }
  }
  // partials: O rows are heads 4 g4 + r, columns dv 16 n + r16
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int hr = 4 * g4 + r;
    if (hr < nh) {
      float* po = p.part_o + (((size_t)b * H + h0 + hr) * p.S + split) * DV;
#pragma unroll
      for (int n = 0; n < NVW; ++n) po[(wv * NVW + n) * 16 + r16] = O[n][r];
    }
  }
  if (g4 == 0 && h_valid && wv == 0) {
    float* pm = p.part_ml + (((size_t)b * H + h) * p.S + split) * 2;
    pm[0] = m;
    pm[1] = l;
  }
}


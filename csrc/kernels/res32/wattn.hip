// Sliding-window attention with a logarithmic distance bias over a paged K/V cache (gfx950, wave64).
//
//   score(i, j) = q_i . k_j - r1_h * ln(1 + r2_h * (i - j))        for 0 <= i - j < window
//   out_i       = softmax_j(score) . v_j
// With a sink (fp32 per head) the softmax's denominator also holds exp(sink_h): a share of the weight that belongs
// to no key and adds no value.
// q arrives in fp32 already multiplied by the head's softmax scale; K rows have D elements, V rows Dv (any sizes,
// D != Dv allowed), G key/value heads serve H query heads (head h reads group h / (H / G)).  Scores, the softmax
// and the weighted sum are fp32 whatever the cache's element type (bf16 or fp32).
//
// Cache layout (one layer): K [num_blocks, block_size, G * D] token rows; V [num_blocks, block_size / 4, G * Dv, 4],
// 4-token interleaved: the four tokens 4t .. 4t+3 of one value column are one 8-byte word (bf16), which is the
// matrix cores' B operand for P V as it lies in memory.  Block strides are given separately (the layers of a model
// share one pool).
//
// Rows are query tokens.  Row t belongs to table row `item`: t itself when cu_q is null (decode: one token
// per sequence), else the item with cu_q[item] <= t < cu_q[item + 1] (a portion of a prompt); its position in
// the sequence is positions[t], and every key it may see is already in the cache.
//
// window_attn_kernel: one wave per (row, head); lanes over 64 keys for the scores, an online softmax per
// 64-key step, then lanes over the value dimension (several keys side by side when Dv < 64).
#include "../common.h"

namespace lwc {
namespace {

template <typename CT> struct KLoad;
template <> struct KLoad<bf16_t> {
  static constexpr int kVec = 8;
  static LWC_DEVICE float dot(const bf16_t* k, const float* q, int D) {
    float acc = 0.f;
    if ((D & 7) == 0 && ((uintptr_t)k & 15) == 0) {
      for (int d = 0; d < D; d += 8) {
        const uint4v kv = *reinterpret_cast<const uint4v*>(k + d);
        float f[8];
        unpack8(kv, f);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += q[d + e] * f[e];
      }
    } else {
      for (int d = 0; d < D; ++d) acc += q[d] * bf2f(k[d]);
    }
    return acc;
  }
  static LWC_DEVICE float ld(const bf16_t* p) { return bf2f(*p); }
  static LWC_DEVICE void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <> struct KLoad<float> {
  static LWC_DEVICE float dot(const float* k, const float* q, int D) {
    float acc = 0.f;
    if ((D & 3) == 0 && ((uintptr_t)k & 15) == 0) {
      for (int d = 0; d < D; d += 4) {
        const float4v kv = *reinterpret_cast<const float4v*>(k + d);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc += q[d + e] * kv[e];
      }
    } else {
      for (int d = 0; d < D; ++d) acc += q[d] * k[d];
    }
    return acc;
  }
  static LWC_DEVICE float ld(const float* p) { return *p; }
  static LWC_DEVICE void st(float* p, float v) { *p = v; }
};

constexpr int kMaxSlots = 8;  // value dimension <= 512

template <typename CT>
__global__ void __launch_bounds__(64)
window_attn_kernel(const float* __restrict__ q, const CT* __restrict__ k_cache, const CT* __restrict__ v_cache,
                   long long kb_stride, long long vb_stride, int block_size, const int* __restrict__ positions,
                   const int* __restrict__ cu_q, int n_items, const int* __restrict__ block_tables, int bt_width,
                   const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ sink, int window,
                   int chunk, CT* __restrict__ out, int ldo, int H, int G, int D, int Dv) {
  extern __shared__ float q_s[];  // [D]
  __shared__ float p_s[64];
  __shared__ long long vo_s[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  int item = t;
  if (cu_q) {
    int lo = 0, hi = n_items - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    item = lo;
  }
  const int* table = block_tables + (size_t)item * bt_width;
  const int i = positions[t];
  const int g = h / (H / G);
  for (int d = lane; d < D; d += 64) q_s[d] = q[((size_t)t * H + h) * D + d];
  __syncthreads();
  const float r1h = r1[h], r2h = r2[h];
  int DvP = 64;
  if (Dv < 64) {
    DvP = 1;
    while (DvP < Dv) DvP <<= 1;
  }
  const int kpar = 64 / DvP, dvl = lane % DvP, kp = lane / DvP;
  float o[kMaxSlots];
#pragma unroll
  for (int ns = 0; ns < kMaxSlots; ++ns) o[ns] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int j_lo = max(max(0, i - window + 1), chunk > 0 ? i - i % chunk : 0);  // the window's and the chunk's first key
  for (int j0 = j_lo; j0 <= i; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= i;
    float s = -INFINITY;
    long long vo = 0;
    if (valid) {
      const long long blk = table[j / block_size];
      const long long off = j % block_size;
      const CT* kr = k_cache + blk * kb_stride + (off * G + g) * D;
      s = KLoad<CT>::dot(kr, q_s, D) - r1h * log1pf(r2h * (float)(i - j));
      vo = blk * vb_stride + (off >> 2) * (4LL * G * Dv) + 4LL * g * Dv + (off & 3);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    vo_s[lane] = vo;
    __syncthreads();
    const int nkeys = min(64, i - j0 + 1);
#pragma unroll
    for (int ns = 0; ns < kMaxSlots; ++ns) o[ns] *= alpha;
    for (int jj = kp; jj < nkeys; jj += kpar) {
      const float pj = p_s[jj];
      const CT* vr = v_cache + vo_s[jj];
#pragma unroll
      for (int ns = 0; ns < kMaxSlots; ++ns) {
        const int dv = ns * 64 + dvl;
        if (dv < Dv) o[ns] += pj * KLoad<CT>::ld(vr + 4 * dv);
      }
    }
  }
  for (int off = DvP; off < 64; off <<= 1) o[0] += __shfl_xor(o[0], off, 64);
  if (sink) {  // a sink: exp(sink_h) joins the denominator; it has no key and no value
    const float sk = sink[h], mf = fmaxf(m, sk), a = expf(m - mf);
    l = l * a + expf(sk - mf);
#pragma unroll
    for (int ns = 0; ns < kMaxSlots; ++ns) o[ns] *= a;
  }
  if (kp == 0) {
    const float inv = 1.0f / l;
    CT* orow = out + (size_t)t * ldo + (size_t)h * Dv;
#pragma unroll
    for (int ns = 0; ns < kMaxSlots; ++ns) {
      const int dv = ns * 64 + dvl;
      if (dv < Dv) KLoad<CT>::st(orow + dv, o[ns] * inv);
    }
  }
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_window_attn(const float* q, const void* k_cache, const void* v_cache, long long kb_stride,
                               long long vb_stride, int block_size, const int* positions, const int* cu_q, int n_items,
                               const int* block_tables, int bt_width, const float* r1, const float* r2, const float* sink,
                               int window, int chunk, void* out, int ldo, int T, int H, int G, int D, int Dv, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (Dv > 64 * kMaxSlots || D > 8192 || H % G != 0) return -1;
  const dim3 grid(T, H);
  const size_t shm = (size_t)D * sizeof(float);
  if (f32)
    window_attn_kernel<float><<<grid, 64, shm, s>>>(q, (const float*)k_cache, (const float*)v_cache, kb_stride, vb_stride,
                                                    block_size, positions, cu_q, n_items, block_tables, bt_width, r1, r2,
                                                    sink, window, chunk, (float*)out, ldo, H, G, D, Dv);
  else
    window_attn_kernel<bf16_t><<<grid, 64, shm, s>>>(q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, kb_stride,
                                                     vb_stride, block_size, positions, cu_q, n_items, block_tables,
                                                     bt_width, r1, r2, sink, window, chunk, (bf16_t*)out, ldo, H, G, D, Dv);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// window_attn_mfma_kernel: prompt portions on the matrix cores (bf16 cache, D = 32 ND, Dv = 16 NV).
//
// Workgroup = 4 waves = 64 consecutive query rows of one (item, head); wave w owns rows 16w .. 16w+15 and all
// four walk the 32-key tiles of the rows' windows, staged through LDS (K row-major; V transposed with the keys
// permuted so that a lane's eight k-slots of one value column are one 16-byte read).  mfma_f32_16x16x32_bf16, lane l:
// r16 = l & 15, g = l >> 4:
//   S^T = K Q^T : A = K rows from LDS, B = Q^T in registers; C reg r = S^T[key 4g + r][query r16], two 16-key
//                 subtiles.  q is fp32: it enters as hi + lo bf16 halves (two MFMAs), so the scores keep fp32's
//                 precision against the cache's bf16 keys.
//   O  += P V   : A = the lane's own softmax weights (k slots 8g+e <-> keys {4g+e, 16+4g+e-4}), again as hi + lo
//                 halves; B = V^T from LDS with the same key permutation; C reg r = O[query 4g + r][dv 16n + r16].
// The distance bias comes from a table bias[h][i - j] (fp32, built once from r1, r2).  Online softmax in fp32;
// masked scores never enter it (weights forced to 0), rows are finite-initialised.
// Positions ascend by one along an item's rows (a portion of a prompt).

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

LWC_DEVICE float4v mfma16(const short8& a, const short8& b, const float4v& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

struct WAttnMfmaParams {
  const float* q;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  long long kb_stride, vb_stride;
  int block_size, bs_shift;  // block_size = 1 << bs_shift (the matrix-core kernels take power-of-two pages)
  const int* positions;
  const int* cu_q;
  const int* k_lens;
  int tiles_per_item;
  const int* block_tables;
  int bt_width;
  const float* bias;  // [H, window], or null: no distance bias
  const float* sink;  // [H], or null: exp(sink_h) joins the softmax denominator of head h (no key, no value)
  int window;
  int chunk;          // > 0: row i sees only keys of its own chunk, j >= i - i % chunk (besides the window)
  bf16_t* out;
  int ldo, H, G;
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kVPad = 40;  // keys per V^T row in LDS (32 + 8: rows stay 16-byte aligned, banks spread)

template <int ND, int NV>
__global__ void __launch_bounds__(256) window_attn_mfma_kernel(const WAttnMfmaParams p) {
  constexpr int D = 32 * ND, DV = 16 * NV, KLD = D + 8;
  constexpr int KCH = (32 * (D / 8) + 255) / 256, VCH = (8 * (DV / 2) + 255) / 256;  // 16-byte words per thread and tile
  // two images of every staged tile: tile kt + 1 is written while tile kt is read (one barrier per tile)
  __shared__ __attribute__((aligned(16))) bf16_t K_s2[2][32 * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vt_s2[2][DV * kVPad];
  __shared__ float bias_s2[2][96];  // the tile's bias by (row - key + 31): rows 0..63 of the workgroup, keys 0..31 of the tile
  extern __shared__ int pages_s[];  // the item's block table over this workgroup's key range (dynamic size)
  // the last row tiles of an item see the most keys: they start first
  const int it = blockIdx.x / p.tiles_per_item, tile = p.tiles_per_item - 1 - blockIdx.x % p.tiles_per_item;
  const int q_begin = p.cu_q[it], q_end = p.cu_q[it + 1];
  const int row0 = q_begin + tile * 64;
  if (row0 >= q_end) return;
  const int h = blockIdx.y, H = p.H, g = h / (H / p.G), G = p.G;
  const int nrows = min(64, q_end - row0);
  const int k_len = p.k_lens[it];
  const int pos0 = p.positions[row0], pos_last = pos0 + nrows - 1;  // positions ascend by one along the rows
  // first visible key of the row at position i: the later of its window's and its chunk's start (ascends with i)
  auto lo_of = [&](int i) { return max(max(0, i - p.window + 1), p.chunk > 0 ? i - i % p.chunk : 0); };
  const int j_lo = lo_of(pos0), j_hi = min(pos_last, k_len - 1);
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, r16 = lane & 15, g4 = lane >> 4;
  const int* table = p.block_tables + (size_t)it * p.bt_width;
  const int BS = p.block_size, bsh = p.bs_shift;
  // page and offset of key j (a runtime division would cost tens of instructions per load)
  auto page_ix = [&](int j) { return j >> bsh; };
  auto page_off = [&](int j) { return j & (BS - 1); };
  typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

  const int qrow = 16 * w + r16;
  const bool q_valid = qrow < nrows;
  const int i_q = pos0 + qrow;
  short8 qhi[ND], qlo[ND];
#pragma unroll
  for (int kd = 0; kd < ND; ++kd) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = 0.f;
      if (q_valid) x = p.q[((size_t)(row0 + qrow) * H + h) * D + kd * 32 + 8 * g4 + e];
      const bf16_t hi = f2bf(x);
      qhi[kd][e] = (short)hi;
      qlo[kd][e] = (short)f2bf(x - bf2f(hi));
    }
  }
  const int w_min = pos0 + 16 * w, w_max = min(pos0 + 16 * w + 15, pos_last);  // this wave's positions
  const int w_lo_min = lo_of(w_min), w_lo_max = lo_of(max(w_max, w_min)), lo_q = lo_of(i_q);  // and their first visible keys
  const bool wave_live = 16 * w < nrows;

  float4v O[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) O[n] = float4v{0.f, 0.f, 0.f, 0.f};
  float m = -1e30f, l = 0.f;
  const float* bias_h = p.bias ? p.bias + (size_t)h * p.window : nullptr;  // no table: no distance bias

  const int pg0 = page_ix((j_lo / 32) * 32);  // first page of the workgroup's key range
  // a tile's words are fetched into registers one tile ahead (the loads fly while the previous tile is computed)
  uint4v kreg[KCH], vreg[VCH];
  float breg = 0.f;
  auto fetch = [&](int kt) {
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int c = tid + 256 * u;
      const int key = c / (D / 8), dc = c % (D / 8);
      const int j = kt * 32 + key;
      kreg[u] = uint4v{0u, 0u, 0u, 0u};
      if (c < 32 * (D / 8) && j <= j_hi) {
        const long long page = pages_s[page_ix(j) - pg0];
        kreg[u] = *reinterpret_cast<const uint4v*>(p.k_cache + page * p.kb_stride + ((long long)page_off(j) * G + g) * D + dc * 8);
      }
    }
    // V: 8 groups of 4 keys; a 16-byte word = 2 value columns x 4 keys
#pragma unroll
    for (int u = 0; u < VCH; ++u) {
      const int c = tid + 256 * u;
      const int kg = c / (DV / 2), dc = c % (DV / 2);
      const int j = kt * 32 + 4 * kg;
      vreg[u] = uint4v{0u, 0u, 0u, 0u};
      if (c < 8 * (DV / 2) && j <= j_hi) {
        const long long page = pages_s[page_ix(j) - pg0];
        vreg[u] = *reinterpret_cast<const uint4v*>(p.v_cache + page * p.vb_stride + (long long)(page_off(j) >> 2) * (4LL * G * DV) +
                                                   4LL * (g * DV + 2 * dc));
      }
    }
    if (tid < 96) {
      const int dist = pos0 - kt * 32 - 31 + tid;  // (row - key + 31) = tid
      breg = bias_h && dist >= 0 && dist < p.window ? bias_h[dist] * kLog2e : 0.f;  // the softmax runs in the log2 domain
    }
  };
  auto stash = [&](int buf) {
    bf16_t* K_s = K_s2[buf];
    bf16_t* Vt_s = Vt_s2[buf];
    float* bias_s = bias_s2[buf];
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int c = tid + 256 * u;
      if (c < 32 * (D / 8)) *reinterpret_cast<uint4v*>(&K_s[(c / (D / 8)) * KLD + (c % (D / 8)) * 8]) = kreg[u];
    }
#pragma unroll
    for (int u = 0; u < VCH; ++u) {
      const int c = tid + 256 * u;
      if (c < 8 * (DV / 2)) {
        const int kg = c / (DV / 2), dc = c % (DV / 2);
        // key group kg (keys 4 kg ..) is k-slots 8 (kg & 3) + 4 (kg >> 2) ..: a lane group's 8 slots lie together
        const int at = 8 * (kg & 3) + 4 * (kg >> 2);
        *reinterpret_cast<uint2v*>(&Vt_s[(2 * dc) * kVPad + at]) = uint2v{vreg[u][0], vreg[u][1]};
        *reinterpret_cast<uint2v*>(&Vt_s[(2 * dc + 1) * kVPad + at]) = uint2v{vreg[u][2], vreg[u][3]};
      }
    }
    if (tid < 96) bias_s[tid] = breg;
  };

  const int kt_lo = j_lo / 32, kt_hi = j_hi / 32;
  // the pages of keys [32 kt_lo, j_hi] once, so a tile's loads do not wait for a table lookup first
  const int npg = page_ix(j_hi) - pg0 + 1;
  for (int c = tid; c < npg; c += 256) pages_s[c] = table[pg0 + c];
  __syncthreads();
  fetch(kt_lo);
  stash(0);
  __syncthreads();
  for (int kt = kt_lo; kt <= kt_hi; ++kt) {
    const int cur = (kt - kt_lo) & 1;
    const bf16_t* K_s = K_s2[cur];
    const bf16_t* Vt_s = Vt_s2[cur];
    const float* bias_s = bias_s2[cur];
    if (kt < kt_hi) fetch(kt + 1);
    // the tile's keys [32 kt, 32 kt + 31] against this wave's rows: nothing visible -> nothing to compute
    if (wave_live && kt * 32 <= w_max && kt * 32 + 31 >= w_lo_min) {
    float4v sacc[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      sacc[sub] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kd = 0; kd < ND; ++kd) {
        const short8 a = *reinterpret_cast<const short8*>(&K_s[(sub * 16 + r16) * KLD + kd * 32 + 8 * g4]);
        sacc[sub] = mfma16(a, qhi[kd], sacc[sub]);
        sacc[sub] = mfma16(a, qlo[kd], sacc[sub]);
      }
    }
    // every key of the tile visible to every row of the wave: no masks
    const bool inner = kt * 32 + 31 <= w_min && kt * 32 >= w_lo_max && w_max - w_min == 15;
    float s[8];
    float mx = -1e30f;
    const float* brow = bias_s + (qrow + 31 - 4 * g4);
    if (inner) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        s[e] = fmaf(sacc[e >> 2][e & 3], kLog2e, -brow[-((e >> 2) * 16 + (e & 3))]);
        mx = fmaxf(mx, s[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int jl = (e >> 2) * 16 + 4 * g4 + (e & 3);
        const int dist = i_q - (kt * 32 + jl);
        const bool ok = q_valid && dist >= 0 && kt * 32 + jl >= lo_q;
        s[e] = ok ? fmaf(sacc[e >> 2][e & 3], kLog2e, -brow[-((e >> 2) * 16 + (e & 3))]) : -1e30f;
        mx = fmaxf(mx, s[e]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    float pe[8], psum = 0.f;
    if (inner) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pe[e] = __builtin_amdgcn_exp2f(s[e] - m_new);
        psum += pe[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pe[e] = s[e] > -1e29f ? __builtin_amdgcn_exp2f(s[e] - m_new) : 0.f;
        psum += pe[e];
      }
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
    // (the running maxima settle after the first tiles: most tiles rescale nothing)
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int n = 0; n < NV; ++n) {
#pragma unroll
        for (int r = 0; r < 4; ++r) O[n][r] *= ar[r];
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const short8 b = *reinterpret_cast<const short8*>(&Vt_s[(n * 16 + r16) * kVPad + 8 * g4]);
      O[n] = mfma16(ph, b, O[n]);
      O[n] = mfma16(pl, b, O[n]);
    }
    }  // (this wave's work on the tile)
    if (kt < kt_hi) stash(cur ^ 1);  // every wave left that image at the previous barrier
    __syncthreads();
  }
  if (!wave_live) return;
  float a_fin = 1.0f;
  if (p.sink) {  // the sink's share: one more term of the denominator, nothing added to O
    const float sk = p.sink[h] * kLog2e, mf = fmaxf(m, sk);
    a_fin = __builtin_amdgcn_exp2f(m - mf);
    l = l * a_fin + __builtin_amdgcn_exp2f(sk - mf);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lr = __shfl(l, 4 * g4 + r, 64);
    const float inv = (lr > 0.f ? 1.0f / lr : 0.f) * __shfl(a_fin, 4 * g4 + r, 64);
    const int row = 16 * w + 4 * g4 + r;
    if (row < nrows) {
      bf16_t* orow = p.out + (size_t)(row0 + row) * p.ldo + (size_t)h * DV;
#pragma unroll
      for (int n = 0; n < NV; ++n) orow[n * 16 + r16] = f2bf(O[n][r] * inv);
    }
  }
}

template <int ND>
int launch_mfma_nv(const WAttnMfmaParams& p, int nv, dim3 grid, size_t shm, hipStream_t s) {
  switch (nv) {
    case 2: window_attn_mfma_kernel<ND, 2><<<grid, 256, shm, s>>>(p); break;
    case 4: window_attn_mfma_kernel<ND, 4><<<grid, 256, shm, s>>>(p); break;
    case 8: window_attn_mfma_kernel<ND, 8><<<grid, 256, shm, s>>>(p); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

// Whether the matrix-core kernel takes these sizes (bf16 cache only).
extern "C" int r32_window_attn_mfma_ok(int D, int Dv) {
  return (D == 32 || D == 64 || D == 128 || D == 192) && (Dv == 32 || Dv == 64 || Dv == 128);
}

extern "C" int r32_window_attn_mfma(const float* q, const void* k_cache, const void* v_cache, long long kb_stride,
                                    long long vb_stride, int block_size, const int* positions, const int* cu_q,
                                    const int* k_lens, int n_items, int max_q, const int* block_tables, int bt_width,
                                    const float* bias, const float* sink, int window, int chunk, void* out, int ldo, int H, int G,
                                    int D, int Dv, hipStream_t s) {
  if (n_items <= 0 || max_q <= 0) return 0;
  if (!r32_window_attn_mfma_ok(D, Dv) || H % G != 0 || (block_size & (block_size - 1)) != 0) return -1;
  WAttnMfmaParams p;
  p.q = q; p.k_cache = (const bf16_t*)k_cache; p.v_cache = (const bf16_t*)v_cache;
  p.kb_stride = kb_stride; p.vb_stride = vb_stride; p.block_size = block_size; p.positions = positions;
  p.bs_shift = -1;
  for (int b = 0; b < 20; ++b)
    if ((1 << b) == block_size) p.bs_shift = b;
  p.cu_q = cu_q; p.k_lens = k_lens; p.tiles_per_item = (max_q + 63) / 64; p.block_tables = block_tables;
  p.bt_width = bt_width; p.bias = bias; p.sink = sink; p.window = window; p.chunk = chunk; p.out = (bf16_t*)out; p.ldo = ldo; p.H = H; p.G = G;
  const dim3 grid(n_items * p.tiles_per_item, H);
  // a workgroup's keys span at most window + 63 positions (from a 32-aligned start: + 31) and never more than the table
  long long span = (long long)window + 63 + 31;
  if (span > (long long)bt_width * block_size) span = (long long)bt_width * block_size;
  const size_t shm = (size_t)(span / block_size + 2) * sizeof(int);
  if (shm > 48 * 1024) return -2;
  switch (D / 32) {
    case 1: return launch_mfma_nv<1>(p, Dv / 16, grid, shm, s);
    case 2: return launch_mfma_nv<2>(p, Dv / 16, grid, shm, s);
    case 4: return launch_mfma_nv<4>(p, Dv / 16, grid, shm, s);
    case 6: return launch_mfma_nv<6>(p, Dv / 16, grid, shm, s);
  }
  return -1;
}

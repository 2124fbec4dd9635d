// Decode rows of the sliding-window attention: the launchers (the kernel is in wattn_decode_kernel.h; the wide
// instantiation is compiled in a file of its own, wattn_decode_wide.hip, with its own code generation flags).
#include "wattn_decode_kernel.h"

// Sizes the decode kernel is built for.  vk: the caller's value pages repeat the first Dv entries of the key rows (a
// latent that is key and value at once); only then does the wide kernel apply (it reads its values from the key rows).
extern "C" int r32_window_attn_decode_ok(int D, int Dv, int vk) {
  const bool small = (D == 32 || D == 64 || D == 128) && (Dv == 32 || Dv == 64 || Dv == 128);
  return small || (vk && D == 576 && Dv == 512);
}

extern "C" int r32_window_attn_decode_wide_launch(const WAttnDecodeParams* p, int gx, int gy, int gz, int chunks_per_group,
                                                  hipStream_t s);

// out[b, h, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s  (splits that saw no key have l = 0)
// sink (or null): exp(sink_h) joins the denominator.
__global__ void window_attn_reduce_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          const float* __restrict__ sink, bf16_t* __restrict__ out, int ldo, int H, int S,
                                          int Dv) {
  const int b = blockIdx.x, h = blockIdx.y;
  const float* ml = part_ml + ((size_t)b * H + h) * S * 2;
  float M = -1e30f;
  for (int s = 0; s < S; ++s)
    if (ml[2 * s + 1] > 0.f) M = fmaxf(M, ml[2 * s]);
  if (sink) M = fmaxf(M, sink[h]);
  float L = sink ? expf(sink[h] - M) : 0.f;
  for (int s = 0; s < S; ++s)
    if (ml[2 * s + 1] > 0.f) L += expf(ml[2 * s] - M) * ml[2 * s + 1];
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  for (int dv = threadIdx.x; dv < Dv; dv += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < S; ++s)
      if (ml[2 * s + 1] > 0.f) acc += expf(ml[2 * s] - M) * part_o[(((size_t)b * H + h) * S + s) * Dv + dv];
    out[(size_t)b * ldo + (size_t)h * Dv + dv] = f2bf(acc * inv);
  }
}

template <int ND>
int launch_decode_nv(const WAttnDecodeParams& p, int nv, dim3 grid, hipStream_t s) {
  switch (nv) {
    case 2: window_attn_decode_kernel<ND, 2><<<grid, 64, 0, s>>>(p); break;
    case 4: window_attn_decode_kernel<ND, 4><<<grid, 64, 0, s>>>(p); break;
    case 8: window_attn_decode_kernel<ND, 8><<<grid, 64, 0, s>>>(p); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

// Splits for a decode step of B sequences whose windows hold at most max_keys keys: about 2048 waves (two per SIMD),
// at least 64 keys each.  Measured at 64 sequences x 8 kv heads x 2048 keys of 128: 3 splits 150 us, 4 splits
// (2048 waves) 130 us, 8 splits 155 us, 16 splits 146 us (shorter key runs per wave, larger partials to merge).
// Wide rows (D = 576): workgroups of four or eight waves, about 512 of them, at least 128 keys each (their partials
// are large).
extern "C" int r32_window_attn_decode_splits(int B, int G, int Hg, int max_keys, int D) {
  const bool wide = D > 128;
  const int chunks = (Hg + 15) / 16;
  const int waves = B * G * (wide && chunks > 1 ? (chunks + 1) / 2 : chunks);  // wide rows: workgroups
  int s = ((wide ? 512 : 2048) + waves - 1) / waves;
  const int by_keys = wide ? (max_keys + 32 + 127) / 128 : (max_keys + 32 + 63) / 64;
  if (s > by_keys) s = by_keys;
  if (s > 64) s = 64;
  return s < 1 ? 1 : s;
}

// part_o: fp32 [B * H * S * Dv], part_ml: fp32 [B * H * S * 2] scratch of the caller.  max_keys: an upper bound of
// the keys any row sees (min(window, longest context)), known on the host.
extern "C" int r32_window_attn_decode(const float* q, const void* k_cache, const void* v_cache, long long kb_stride,
                                      long long vb_stride, int block_size, const int* positions, const int* block_tables,
                                      int bt_width, const float* bias, const float* sink, int window, int chunk, float* part_o,
                                      float* part_ml, int S, int max_keys, void* out, int ldo, int B, int H, int G, int D,
                                      int Dv, int vk, hipStream_t s) {
  if (B <= 0) return 0;
  if (!r32_window_attn_decode_ok(D, Dv, vk) || H % G != 0 || S < 1 || (block_size & (block_size - 1)) != 0) return -1;
  WAttnDecodeParams p;
  p.q = q; p.k_cache = (const bf16_t*)k_cache; p.v_cache = (const bf16_t*)v_cache; p.kb_stride = kb_stride;
  p.vb_stride = vb_stride; p.block_size = block_size; p.positions = positions; p.block_tables = block_tables;
  p.bs_shift = -1;
  for (int b = 0; b < 20; ++b)
    if ((1 << b) == block_size) p.bs_shift = b;
  p.bt_width = bt_width; p.bias = bias; p.window = window; p.chunk = chunk; p.part_o = part_o; p.part_ml = part_ml; p.H = H; p.G = G;
  p.S = S;
  // a row's keys start at a multiple of 32 at or below its window's first key: up to max_keys + 31 keys to cover
  p.keys_per_split = (((max_keys + 31 + S - 1) / S) + 31) / 32 * 32;
  const int Hg = H / G;
  const dim3 grid(B, G * ((Hg + 15) / 16), S);
  int rc = -1;
  if (D == 576 && Dv == 512) {  // one wide row for all heads: a low-rank attention's cached latent + rotated part
    const int chunks = (Hg + 15) / 16, nc = chunks > 1 ? 2 : 1;  // more than 16 heads: two chunks per workgroup
    rc = r32_window_attn_decode_wide_launch(&p, B, G * ((chunks + nc - 1) / nc), S, nc, s);
  } else {
    switch (D / 32) {
      case 1: rc = launch_decode_nv<1>(p, Dv / 16, grid, s); break;
      case 2: rc = launch_decode_nv<2>(p, Dv / 16, grid, s); break;
      case 4: rc = launch_decode_nv<4>(p, Dv / 16, grid, s); break;
    }
  }
  if (rc != 0) return rc;
  window_attn_reduce_kernel<<<dim3(B, H), 64, 0, s>>>(part_o, part_ml, sink, (bf16_t*)out, ldo, H, S, Dv);
  return (int)hipGetLastError();
}

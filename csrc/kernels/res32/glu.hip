// Gated feed-forward activations over fused [gate | up] rows (gfx950, wave64); arithmetic fp32.
//
//   mode 0   y = silu(g) * u
//   mode 1   g' = min(g, L), u' = clamp(u, -L, L);  y = g' * sigmoid(alpha g') * (u' + 1)      (clamped gate unit)
// in: rows [gate (n) | up (n)] with leading dimension ldi; out: rows of n (leading dimension ldo).
//
//   gelu     y = z / 2 (1 + erf(z / sqrt(2))) over rows of n (an ungated feed-forward's activation)
#include "elem.h"

namespace lwc {
namespace {

template <int MODE> LWC_DEVICE float glu_f(float g, float u, float alpha, float limit) {
  if (MODE == 0) return silu_f(g) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoid_f(alpha * g) * (u + 1.0f);
}

template <typename AT, int MODE>
__global__ void glu_kernel(const AT* __restrict__ in, int ldi, AT* __restrict__ out, int ldo, int n, long long total,
                           float alpha, float limit) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    const long long t = e / n;
    const int c = (int)(e - t * n);
    const AT* r = in + t * ldi;
    Elem<AT>::st(out + t * ldo + c, glu_f<MODE>(Elem<AT>::ld(r + c), Elem<AT>::ld(r + n + c), alpha, limit));
  }
}

// four columns per thread: n, ldi, ldo multiples of four and aligned bases
template <typename AT, int MODE>
__global__ void glu_vec_kernel(const AT* __restrict__ in, int ldi, AT* __restrict__ out, int ldo, int n4, long long total4,
                               float alpha, float limit) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total4; e += (long long)gridDim.x * blockDim.x) {
    const long long t = e / n4;
    const int c = 4 * (int)(e - t * n4);
    const AT* r = in + t * ldi;
    const float4v g = Vec4<AT>::ld(r + c), u = Vec4<AT>::ld(r + 4 * n4 + c);
    Vec4<AT>::st(out + t * ldo + c, float4v{glu_f<MODE>(g[0], u[0], alpha, limit), glu_f<MODE>(g[1], u[1], alpha, limit),
                                            glu_f<MODE>(g[2], u[2], alpha, limit), glu_f<MODE>(g[3], u[3], alpha, limit)});
  }
}

// Gelu<AT>: the erf form.  fp32 rows: the library's erff.  bf16 rows: erf by the rational form 1 - (a1 t + ... + a5 t^5)
// exp(-x^2), t = 1 / (1 + p x) (Abramowitz and Stegun 7.1.26; absolute error 1.5e-7, far below a bf16 result's
// rounding), a third of the instructions.
template <typename AT> struct Gelu {
  static LWC_DEVICE float f(float z) { return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f)); }
};
template <> struct Gelu<bf16_t> {
  static LWC_DEVICE float f(float z) {
    const float x = fabsf(z) * 0.7071067811865476f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, x, 1.0f));
    const float p = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float e = 1.0f - p * __expf(-x * x);
    return 0.5f * z * (1.0f + copysignf(e, z));
  }
};

template <typename AT>
__global__ void gelu_kernel(const AT* __restrict__ in, int ldi, AT* __restrict__ out, int ldo, int n, long long total) {
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    const long long t = e / n;
    const int c = (int)(e - t * n);
    Elem<AT>::st(out + t * ldo + c, Gelu<AT>::f(Elem<AT>::ld(in + t * ldi + c)));
  }
}

// four columns per thread, rows along the grid's second dimension (no division per element)
template <typename AT>
__global__ void gelu_vec_kernel(const AT* __restrict__ in, int ldi, AT* __restrict__ out, int ldo, int n4, int T) {
  const int c = 4 * (blockIdx.x * blockDim.x + threadIdx.x);
  if (c >= 4 * n4) return;
  for (int t = blockIdx.y; t < T; t += gridDim.y) {
    const float4v z = Vec4<AT>::ld(in + (size_t)t * ldi + c);
    Vec4<AT>::st(out + (size_t)t * ldo + c, float4v{Gelu<AT>::f(z[0]), Gelu<AT>::f(z[1]), Gelu<AT>::f(z[2]), Gelu<AT>::f(z[3])});
  }
}

int glu_grid(long long total) {
  const long long g = (total + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace
}  // namespace lwc

using namespace lwc;

extern "C" int r32_glu(const void* in, int ldi, void* out, int ldo, int T, int n, int mode, float alpha, float limit, int f32,
                       hipStream_t s) {
  const long long total = (long long)T * n;
  if (total <= 0) return 0;
  if (mode != 0 && mode != 1) return -1;
  const int ab = f32 ? 16 : 8;
  const bool vec = n % 4 == 0 && ldi % 4 == 0 && ldo % 4 == 0 && aligned_to(in, ab) && aligned_to(out, ab);
#define LWC_GLU(AT, M)                                                                                                   \
  if (vec)                                                                                                               \
    glu_vec_kernel<AT, M><<<glu_grid(total / 4), 256, 0, s>>>((const AT*)in, ldi, (AT*)out, ldo, n / 4, total / 4, alpha, \
                                                              limit);                                                    \
  else                                                                                                                   \
    glu_kernel<AT, M><<<glu_grid(total), 256, 0, s>>>((const AT*)in, ldi, (AT*)out, ldo, n, total, alpha, limit)
  if (f32) {
    if (mode == 0) {
      LWC_GLU(float, 0);
    } else {
      LWC_GLU(float, 1);
    }
  } else {
    if (mode == 0) {
      LWC_GLU(bf16_t, 0);
    } else {
      LWC_GLU(bf16_t, 1);
    }
  }
#undef LWC_GLU
  LWC_CHECK_LAUNCH();
  return 0;
}

extern "C" int r32_gelu(const void* in, int ldi, void* out, int ldo, int T, int n, int f32, hipStream_t s) {
  const long long total = (long long)T * n;
  if (total <= 0) return 0;
  const int ab = f32 ? 16 : 8;
  const bool vec = n % 4 == 0 && ldi % 4 == 0 && ldo % 4 == 0 && aligned_to(in, ab) && aligned_to(out, ab);
  const dim3 vgrid((n / 4 + 255) / 256, T < 32768 ? T : 32768);
  if (vec && f32) gelu_vec_kernel<float><<<vgrid, 256, 0, s>>>((const float*)in, ldi, (float*)out, ldo, n / 4, T);
  else if (vec) gelu_vec_kernel<bf16_t><<<vgrid, 256, 0, s>>>((const bf16_t*)in, ldi, (bf16_t*)out, ldo, n / 4, T);
  else if (f32) gelu_kernel<float><<<glu_grid(total), 256, 0, s>>>((const float*)in, ldi, (float*)out, ldo, n, total);
  else gelu_kernel<bf16_t><<<glu_grid(total), 256, 0, s>>>((const bf16_t*)in, ldi, (bf16_t*)out, ldo, n, total);
  LWC_CHECK_LAUNCH();
  return 0;
}

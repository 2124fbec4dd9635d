// The decode kernel for ONE wide cached row shared by all heads (576 key entries, 512 value entries: a low-rank
// attention's latent + rotated part): four waves per workgroup, key rows through LDS, q as its bf16 rounding.  A file
// of its own so that it gets its own code generation flags (accumulators kept in VGPRs).
#include "wattn_decode_kernel.h"

extern "C" int r32_window_attn_decode_wide_launch(const WAttnDecodeParams* p, int gx, int gy, int gz, hipStream_t s) {
  window_attn_decode_kernel<18, 32, 4, false><<<dim3(gx, gy, gz), 256, 0, s>>>(*p);
  return (int)hipGetLastError();
}

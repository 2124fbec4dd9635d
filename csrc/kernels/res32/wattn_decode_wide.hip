// The decode kernel for ONE wide cached row shared by all heads (576 key entries, 512 value entries: a low-rank
// attention's latent + rotated part): four waves per workgroup, key rows through LDS, the value operands gathered from
// those rows (the latent is key and value at once; the caller guarantees that the value pages repeat the key rows'
// first 512 entries), q as its bf16 rounding.  A file
// of its own so that it gets its own code generation flags (accumulators kept in VGPRs).
#include "wattn_decode_kernel.h"

// chunks_per_group 2: two 16-head chunks share a workgroup (eight waves) and its staged key rows; gy counts workgroups
extern "C" int r32_window_attn_decode_wide_launch(const WAttnDecodeParams* p, int gx, int gy, int gz, int chunks_per_group,
                                                  hipStream_t s) {
  if (chunks_per_group == 2) window_attn_decode_kernel<18, 32, 4, false, true, 2><<<dim3(gx, gy, gz), 512, 0, s>>>(*p);
  else window_attn_decode_kernel<18, 32, 4, false, true, 1><<<dim3(gx, gy, gz), 256, 0, s>>>(*p);
  return (int)hipGetLastError();
}

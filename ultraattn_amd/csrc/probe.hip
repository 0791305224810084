// Diagnostic: sustained rate of back-to-back v_mfma_f32_32x32x16_bf16 from registers only (no LDS,
// no memory traffic), with constant or random operand bits.  The shader clock of this part
// follows the power drawn, and the power of the matrix pipe follows the bit activity of its
// operands, so the two rates differ; the random-data rate is the practical ceiling for any
// bf16 MFMA kernel fed with ordinary data.
#include "ua_common.h"

namespace ua {

__global__ __launch_bounds__(256) void probe_mfma_kernel(const u32x4* in, float* out, int iters) {
  const u32x4 ra = in[threadIdx.x], rb = in[256 + threadIdx.x];
  bf16x8 a, b;
  __builtin_memcpy(&a, &ra, 16);
  __builtin_memcpy(&b, &rb, 16);
  f32x16 c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = f32x16{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = mfma32(a, b, c[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += c[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace ua

extern "C" int ua_probe_mfma(const void* operands, float* out, int n_blocks, int iters, void* stream) {
  using namespace ua;
  if (!operands || !out) return UA_ERR_NULL;
  if (n_blocks <= 0 || iters <= 0) return UA_ERR_SHAPE;
  if (!aligned16(operands)) return UA_ERR_ALIGN;
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(n_blocks), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)operands, out, iters);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

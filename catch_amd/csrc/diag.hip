// Measurement aid behind the C ABI: the rate the int8 matrix cores sustain on this device when nothing else
// limits them.  A register-resident loop of v_mfma_i32_32x32x32_i8 with four independent accumulators per wave
// and no memory access inside the loop; the operands are whatever the caller put into `operands`, because the
// rate depends on them: the device lowers its clock under high-toggle matrix work.
#include "catchq_common.h"

namespace catchq {

__global__ __launch_bounds__(256) void mfma_loop_kernel(const v4i *__restrict__ operands, int iters, int *sink) {
  // eight operand fragments per lane, read once
  v4i a[4], b[4];
  const int lane = blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(lane * 8 + i) & 0xffff];
    b[i] = operands[(lane * 8 + 4 + i) & 0xffff];
  }
  v16i c[4] = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[(i + it) & 3], c[i], 0, 0, 0);
  }
  int r = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) r += c[i][j];
  if (r == 0x7f123456) sink[0] = r;  // keeps the loop alive
}

}  // namespace catchq

using namespace catchq;

CATCHQ_API int catchq_diag_mfma_i8_loop(const void *operands, int iters, int blocks, int32_t *sink,
                                        catchq_stream_t stream) {
  if (!operands || !sink || iters < 0 || blocks < 1 || blocks > (1 << 20) || !aligned16(operands)) return CATCHQ_ERR_ARG;
  mfma_loop_kernel<<<blocks, 256, 0, as_stream(stream)>>>((const v4i *)operands, iters, sink);
  return launch_status();
}

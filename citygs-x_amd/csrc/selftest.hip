// Device self-test of the cross-lane reduction primitives used by the blend
// kernels, so their lane semantics can be checked against plain sums.
#include "gs_common.h"
#include "gs_kernels.h"
#include "render_common.h"

namespace gs {

namespace {

// in: [64 lanes][16 values]; out_wave[16] = sums over the 64 lanes;
// out_rows[4][16] = sums over each 16-lane row.
__global__ void __launch_bounds__(GS_WAVE) reduce_selftest_kernel(const float* __restrict__ in,
                                                                  float* __restrict__ out_wave,
                                                                  float* __restrict__ out_rows) {
  const int lane = threadIdx.x;
  float v[16];
#pragma unroll
  for (int q = 0; q < 16; q++) v[q] = in[lane * 16 + q];
  float r[4];
  wave_reduce16(v, r);
  if ((lane & 15) == 0) {
    const int row = lane >> 4;
#pragma unroll
    for (int k = 0; k < 4; k++) out_wave[k + 4 * row] = r[k];
  }
  const float t = row_transpose_reduce16(v);
  out_rows[(lane >> 4) * 16 + (lane & 15)] = t;
}

}  // namespace

int launch_reduce_selftest(const float* in, float* out_wave, float* out_rows, hipStream_t stream) {
  hipLaunchKernelGGL(reduce_selftest_kernel, dim3(1), dim3(GS_WAVE), 0, stream, in, out_wave, out_rows);
  return 0;
}

}  // namespace gs

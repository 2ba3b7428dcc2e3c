// Per-Gaussian geometry channels of the blend ("all_map": camera-space normal, 1, plane distance) and
// their backward pass: the torch lines of gaussian_renderer/__init__.py:1501-1518 (quaternion_to_matrix
// of pytorch3d 0.3.0 on the normalised rotation, the axis of the smallest scale as normal, flipped
// towards the camera, rotated into the camera frame, distance = |normal . p_cam|) as one streaming
// kernel each way instead of about ten elementwise launches.  One thread per Gaussian; 40 bytes in and
// 20 out forward, 60 in and 28 out backward.  Sums run left to right with one rounding per operation.
#include "all_map_common.h"
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

__global__ void __launch_bounds__(GS_BLOCK_1D)
all_map_fwd_kernel(int P, const float* __restrict__ means, const float* __restrict__ scales,
                   const float* __restrict__ rots, const float* __restrict__ Vg, const float* __restrict__ camg,
                   float* __restrict__ out) {
  // the workgroup's 256 rows of 5 floats leave through LDS as 1280 consecutive floats (20-byte rows written
  // lane by lane would touch every line five times)
  __shared__ float s_out[5 * GS_BLOCK_1D];
  const int raw = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  const int i = raw < P ? raw : P - 1;
  float V[16], cam[3];
#pragma unroll
  for (int k = 0; k < 16; k++) V[k] = Vg[k];
#pragma unroll
  for (int k = 0; k < 3; k++) cam[k] = camg[k];
  const float m[3] = {means[3 * (size_t)i], means[3 * (size_t)i + 1], means[3 * (size_t)i + 2]};
  const float s[3] = {scales[3 * (size_t)i], scales[3 * (size_t)i + 1], scales[3 * (size_t)i + 2]};
  AllMapGeom g;
  all_map_geom(m, s, reinterpret_cast<const float4*>(rots)[i], V, cam, g);
  all_map_channels(g, s_out + 5 * threadIdx.x);
  __syncthreads();
  const size_t first = 5 * (size_t)blockIdx.x * GS_BLOCK_1D, total = 5 * (size_t)P;
#pragma unroll
  for (int k = 0; k < 5; k++) {
    const size_t e = first + (size_t)k * GS_BLOCK_1D + threadIdx.x;
    if (e < total) out[e] = s_out[k * GS_BLOCK_1D + threadIdx.x];
  }
}

__global__ void __launch_bounds__(GS_BLOCK_1D)
all_map_bwd_kernel(int P, const float* __restrict__ means, const float* __restrict__ scales,
                   const float* __restrict__ rots, const float* __restrict__ Vg, const float* __restrict__ camg,
                   const float* __restrict__ gout, float* __restrict__ dmeans, float* __restrict__ drots) {
  const int idx = blockIdx.x * GS_BLOCK_1D + threadIdx.x;
  if (idx >= P) return;
  float V[16], cam[3];
#pragma unroll
  for (int k = 0; k < 16; k++) V[k] = Vg[k];
#pragma unroll
  for (int k = 0; k < 3; k++) cam[k] = camg[k];
  const float m[3] = {means[3 * (size_t)idx], means[3 * (size_t)idx + 1], means[3 * (size_t)idx + 2]};
  const float s[3] = {scales[3 * (size_t)idx], scales[3 * (size_t)idx + 1], scales[3 * (size_t)idx + 2]};
  AllMapGeom g;
  all_map_geom(m, s, reinterpret_cast<const float4*>(rots)[idx], V, cam, g);
  const float* go = gout + 5 * (size_t)idx;
  const float g0 = go[0], g1 = go[1], g2 = go[2], g4 = go[4];
  const float sdot = (g.loc[0] * g.pc[0] + g.loc[1] * g.pc[1]) + g.loc[2] * g.pc[2];
  const float gs_ = g4 * (sdot > 0.0f ? 1.0f : (sdot < 0.0f ? -1.0f : 0.0f));  // d|s| = sign(s)
  const float gl[3] = {g0 + gs_ * g.pc[0], g1 + gs_ * g.pc[1], g2 + gs_ * g.pc[2]};
  const float gp[3] = {gs_ * g.loc[0], gs_ * g.loc[1], gs_ * g.loc[2]};
  float gn[3];
#pragma unroll
  for (int a = 0; a < 3; a++) {
    gn[a] = g.sgn * ((gl[0] * V[4 * a] + gl[1] * V[4 * a + 1]) + gl[2] * V[4 * a + 2]);
    dmeans[3 * (size_t)idx + a] = (gp[0] * V[4 * a] + gp[1] * V[4 * a + 1]) + gp[2] * V[4 * a + 2];
  }
  // the chosen column of R as a function of (r,i,j,k) and two_s = 2/(q.q)
  const float r = g.q[0], i = g.q[1], j = g.q[2], k = g.q[3], ts = g.two_s;
  float gq[4], gts;
  if (g.axis == 0) {
    gq[0] = ts * (k * gn[1] - j * gn[2]);
    gq[1] = ts * (j * gn[1] + k * gn[2]);
    gq[2] = ts * ((-2.0f * j * gn[0] + i * gn[1]) - r * gn[2]);
    gq[3] = ts * ((-2.0f * k * gn[0] + r * gn[1]) + i * gn[2]);
    gts = (-(j * j + k * k) * gn[0] + (i * j + k * r) * gn[1]) + (i * k - j * r) * gn[2];
  } else if (g.axis == 1) {
    gq[0] = ts * (-k * gn[0] + i * gn[2]);
    gq[1] = ts * ((j * gn[0] - 2.0f * i * gn[1]) + r * gn[2]);
    gq[2] = ts * (i * gn[0] + k * gn[2]);
    gq[3] = ts * ((-r * gn[0] - 2.0f * k * gn[1]) + j * gn[2]);
    gts = ((i * j - k * r) * gn[0] - (i * i + k * k) * gn[1]) + (j * k + i * r) * gn[2];
  } else {
    gq[0] = ts * (j * gn[0] - i * gn[1]);
    gq[1] = ts * ((k * gn[0] - r * gn[1]) - 2.0f * i * gn[2]);
    gq[2] = ts * ((r * gn[0] + k * gn[1]) - 2.0f * j * gn[2]);
    gq[3] = ts * (i * gn[0] + j * gn[1]);
    gts = ((i * k + j * r) * gn[0] + (j * k - i * r) * gn[1]) - (i * i + j * j) * gn[2];
  }
  const float w = -(ts * ts) * gts;  // d two_s / dq = -two_s^2 q
#pragma unroll
  for (int a = 0; a < 4; a++) gq[a] += w * g.q[a];
  // backward of q / max(|q|, eps)
  float dq[4];
  if (g.len > 1e-12f) {
    const float dot = ((g.q[0] * gq[0] + g.q[1] * gq[1]) + g.q[2] * gq[2]) + g.q[3] * gq[3];
#pragma unroll
    for (int a = 0; a < 4; a++) dq[a] = (gq[a] - g.q[a] * dot) / g.len;
  } else {
    const float den = fmaxf(g.len, 1e-12f);
#pragma unroll
    for (int a = 0; a < 4; a++) dq[a] = gq[a] / den;
  }
  reinterpret_cast<float4*>(drots)[idx] = make_float4(dq[0], dq[1], dq[2], dq[3]);
}

}  // namespace

int launch_all_map_fwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                       const float* campos, float* out, hipStream_t stream) {
  if (P <= 0) return 0;
  hipLaunchKernelGGL(all_map_fwd_kernel, dim3((P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0, stream, P,
                     means, scales, rots, V, campos, out);
  return 0;
}

int launch_all_map_bwd(int P, const float* means, const float* scales, const float* rots, const float* V,
                       const float* campos, const float* grad_out, float* dmeans, float* drots,
                       hipStream_t stream) {
  if (P <= 0) return 0;
  hipLaunchKernelGGL(all_map_bwd_kernel, dim3((P + GS_BLOCK_1D - 1) / GS_BLOCK_1D), dim3(GS_BLOCK_1D), 0, stream, P,
                     means, scales, rots, V, campos, grad_out, dmeans, drots);
  return 0;
}

}  // namespace gs

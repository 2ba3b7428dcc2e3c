// The per-Gaussian geometry channels of the blend ("all_map": camera-space normal, 1, plane distance): what the
// all_map kernels and the preprocess kernel (when it writes the blend kernels' operand records) share, so that
// both form the same bits from the same inputs.
#pragma once

#include "gs_common.h"

namespace gs {

struct AllMapGeom {
  float q[4];     // normalised rotation
  float len;      // |q| before normalisation
  float two_s;    // 2 / (q.q)
  int axis;       // column of the rotation matrix that serves as normal
  float sgn;      // -1 when the normal was flipped towards the camera
  float loc[3];   // normal in the camera frame
  float pc[3];    // centre in the camera frame
};

__device__ __forceinline__ void rot_column(const float* q, int c, float ts, float* n) {
  const float r = q[0], i = q[1], j = q[2], k = q[3];
  if (c == 0) {
    n[0] = 1.0f - ts * (j * j + k * k);
    n[1] = ts * (i * j + k * r);
    n[2] = ts * (i * k - j * r);
  } else if (c == 1) {
    n[0] = ts * (i * j - k * r);
    n[1] = 1.0f - ts * (i * i + k * k);
    n[2] = ts * (j * k + i * r);
  } else {
    n[0] = ts * (i * k + j * r);
    n[1] = ts * (j * k - i * r);
    n[2] = 1.0f - ts * (i * i + j * j);
  }
}

__device__ __forceinline__ void all_map_geom(const float* m, const float* s, float4 q0, const float* V,
                                             const float* cam, AllMapGeom& g) {
  g.len = sqrtf(((q0.x * q0.x + q0.y * q0.y) + q0.z * q0.z) + q0.w * q0.w);
  const float den = fmaxf(g.len, 1e-12f);  // torch.nn.functional.normalize(eps=1e-12)
  g.q[0] = q0.x / den; g.q[1] = q0.y / den; g.q[2] = q0.z / den; g.q[3] = q0.w / den;
  g.two_s = 2.0f / (((g.q[0] * g.q[0] + g.q[1] * g.q[1]) + g.q[2] * g.q[2]) + g.q[3] * g.q[3]);
  int a = 0;
  if (s[1] < s[a]) a = 1;
  if (s[2] < s[a]) a = 2;
  g.axis = a;
  float n[3];
  rot_column(g.q, a, g.two_s, n);
  const float tc[3] = {cam[0] - m[0], cam[1] - m[1], cam[2] - m[2]};
  g.sgn = ((n[0] * tc[0] + n[1] * tc[1]) + n[2] * tc[2] < 0.0f) ? -1.0f : 1.0f;
#pragma unroll
  for (int k = 0; k < 3; k++) {
    g.loc[k] = g.sgn * ((n[0] * V[k] + n[1] * V[4 + k]) + n[2] * V[8 + k]);
    g.pc[k] = ((m[0] * V[k] + m[1] * V[4 + k]) + m[2] * V[8 + k]) + V[12 + k];
  }
}

// The five channels [normal_cam(3), 1, |normal . p_cam|] (gaussian_renderer/__init__.py:1501-1518).
__device__ __forceinline__ void all_map_channels(const AllMapGeom& g, float* o) {
  o[0] = g.loc[0];
  o[1] = g.loc[1];
  o[2] = g.loc[2];
  o[3] = 1.0f;
  o[4] = fabsf((g.loc[0] * g.pc[0] + g.loc[1] * g.pc[1]) + g.loc[2] * g.pc[2]);
}

}  // namespace gs

// Pieces shared by the forward and backward tile kernels: the pixel layout of a
// workgroup, the conservative screen-space bounding box used to cull Gaussians
// per wave, and the 64-lane reduction of 16 values.
#pragma once

#include "gs_common.h"

namespace gs {

// A 16x16 tile is rendered by 256 threads = four 64-lane waves; each wave owns
// an 8x8 quadrant (lane = 8*row + column inside the quadrant).  Compared with
// 16x4 strips this keeps a wave's pixels compact, so fewer Gaussians of the
// tile's list overlap any given wave.
struct TileThread {
  int lane, wave;
  uint32_t px, py;    // this thread's pixel
  float wx0, wy0, wx1, wy1;  // the wave's pixel rectangle (inclusive), as floats
};

__device__ __forceinline__ TileThread tile_thread(uint32_t tile_x, uint32_t tile_y) {
  TileThread t;
  const int tid = threadIdx.x;
  t.lane = tid & (GS_WAVE - 1);
  t.wave = tid / GS_WAVE;
  const uint32_t qx = (uint32_t)(t.wave & 1) * 8u, qy = (uint32_t)(t.wave >> 1) * 8u;
  const uint32_t x0 = tile_x * GS_TILE_X + qx, y0 = tile_y * GS_TILE_Y + qy;
  t.px = x0 + (uint32_t)(t.lane & 7);
  t.py = y0 + (uint32_t)(t.lane >> 3);
  t.wx0 = (float)x0;
  t.wy0 = (float)y0;
  t.wx1 = (float)(x0 + 7u);
  t.wy1 = (float)(y0 + 7u);
  return t;
}

// Axis-aligned box outside of which a Gaussian cannot pass the blend tests of
// cuda_rasterizer/forward.cu:381-393 (power <= 0 and opacity*exp(power) >= 1/255).
// With conic (A,B,C) and tau = ln(255*opacity), alpha >= 1/255 needs
// A dx^2 + 2B dx dy + C dy^2 <= 2 tau, whose extent along x is sqrt(2 tau C / (AC-B^2)).
// The box is inflated (tau + 0.01, then 0.1 % and half a pixel) so that fp32
// rounding in the per-pixel evaluation can never disagree with it; whenever the
// box cannot be trusted (non-positive determinant, NaN) it is infinite.  Culling
// with it only skips work, it never changes a result.
// power_floor receives the exponent below which alpha < 1/255 is certain (never below -87, where
// gs_expf returns 0 anyway): pixels with power < power_floor can skip the exponential.
__device__ __forceinline__ float4 cull_box(float2 xy, float4 co, float& power_floor) {
  const float inf = __builtin_inff();
  float4 bb = make_float4(-inf, -inf, inf, inf);  // xmin, ymin, xmax, ymax
  const float o = co.w;
  power_floor = -87.0f;
  if (o < 0.0039f) {
    // opacity below 1/255: alpha = o*exp(power) with power <= 0 can never reach 1/255
    return make_float4(inf, inf, -inf, -inf);
  }
  const float det = co.x * co.z - co.y * co.y;
  if (o < 1.0e30f) {
    const float tau = __logf(255.0f * o) + 0.01f;
    if (tau == tau) power_floor = fmaxf(-tau, -87.0f);
  }
  if (det > 0.0f && o < 1.0e30f) {
    const float tau = __logf(255.0f * o) + 0.01f;
    const float s = 2.0f * tau / det;
    const float ex = sqrtf(s * co.z) * 1.001f + 0.5f;
    const float ey = sqrtf(s * co.x) * 1.001f + 0.5f;
    if (ex == ex && ey == ey) bb = make_float4(xy.x - ex, xy.y - ey, xy.x + ex, xy.y + ey);
  }
  return bb;
}

__device__ __forceinline__ bool box_hits_wave(const float4 bb, const TileThread& t) {
  return !(bb.z < t.wx0 || bb.x > t.wx1 || bb.w < t.wy0 || bb.y > t.wy1);
}

template <int CTRL>
__device__ __forceinline__ float dpp_row_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
  return v + __int_as_float(moved);
}

// Sums 16 per-lane values over the 64 lanes of a wave in 40 operations.
//   level 1: v_permlane32_swap pairs value k with k+8: the low 32 lanes keep k, the high 32 lanes k+8;
//   level 2: v_permlane16_swap pairs k with k+4: each 16-lane row keeps one value;
//   level 3: four DPP adds (quad swaps, row rotations) finish the sum inside each row.
// On return every lane of row r (lanes 16r..16r+15) of out[k] holds the total of value k + 4r.
__device__ __forceinline__ void wave_reduce16(const float* v, float* out) {
  float h[8];
#pragma unroll
  for (int k = 0; k < 8; k++) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[k]), __float_as_uint(v[k + 8]), false, false);
    h[k] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  }
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(h[k]), __float_as_uint(h[k + 4]), false, false);
    float s = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    s = dpp_row_add<0xB1>(s);   // quad_perm [1,0,3,2]
    s = dpp_row_add<0x4E>(s);   // quad_perm [2,3,0,1]
    s = dpp_row_add<0x124>(s);  // row_ror:4
    s = dpp_row_add<0x128>(s);  // row_ror:8
    out[k] = s;
  }
}

}  // namespace gs

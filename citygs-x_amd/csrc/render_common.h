// Pieces shared by the forward and backward tile kernels: the pixel layout of a
// workgroup, the conservative test that culls Gaussians per 4x4 pixel block, and
// the reductions of 16 values over a wave and over a 16-lane row.
#pragma once

#include "gs_common.h"

namespace gs {

// Which Gaussians can pass the blend tests of cuda_rasterizer/forward.cu:381-393 (power <= 0 and
// opacity * exp(power) >= 1/255) somewhere in a block of pixels.  With conic (A, B, C) and
// tau = ln(255 * opacity), alpha >= 1/255 needs q(d) = A dx^2 + 2 B dx dy + C dy^2 <= 2 tau.
// cull_params returns (1/A, 1/C, q_max, 0) with q_max = 2 (tau + 0.01).  q_max is +infinity when the conic
// cannot be trusted (every block then counts as hit) and negative when the opacity alone rules every pixel out.
// power_floor receives the exponent below which alpha < 1/255 is certain (never below -87, where gs_expf
// returns 0 anyway): pixels with power < power_floor can skip the exponential.  Culling with these only skips
// work, it never changes a result.
__device__ __forceinline__ float4 cull_params(float4 co, float& power_floor) {
  const float inf = __builtin_inff();
  const float o = co.w;
  power_floor = -87.0f;
  if (o < 0.0039f) return make_float4(0.f, 0.f, -1.0f, 0.f);
  float4 cp = make_float4(0.f, 0.f, inf, 0.f);
  if (o < 1.0e30f) {
    const float tau = __logf(255.0f * o) + 0.01f;
    if (tau == tau) {
      power_floor = fmaxf(-tau, -87.0f);
      const float det = co.x * co.z - co.y * co.y;
      // (the hardware reciprocal: 1/A and 1/C only place the point of a block edge where q is evaluated, and q
      // there exceeds the edge's minimum by the square of the placement error)
      const float ia = __builtin_amdgcn_rcpf(co.x), ic = __builtin_amdgcn_rcpf(co.z);
      if (det > 0.0f && co.x > 0.0f && co.z > 0.0f && ia < inf && ic < inf) cp = make_float4(ia, ic, 2.0f * tau, 0.f);
    }
  }
  return cp;
}

// What the block tests of a tile's kernels need of a Gaussian centred at xy: (1/A, 1/C, limit on q, 0), and, in
// mark_limit, the limit on q for a single pixel of the tile (the forward blend marks the pixels an entry can reach
// with it).  Both limits are q_max plus a margin for rounding: the block test, the pixel mark and the blend itself
// evaluate q by different operation sequences at different points, each within a few units in the last place of
// the LARGEST term, which for a long thin Gaussian far from its centre is much larger than q itself.  Every such
// term is at most S = A X^2 + 2 |B| X Y + C Y^2 with X, Y the largest offsets of a pixel of the tile from the
// centre; the margin is 2e-6 S (about 32 units in the last place of S), on top of the 0.02 from tau + 0.01.  The
// block limit is negative when the opacity alone rules every pixel out and +infinity when the conic cannot be
// trusted.  The same numbers in the forward and the backward kernel, so both build the same lists.
__device__ __forceinline__ float4 block_test_params(float4 co, float2 xy, float tile_x0, float tile_y0,
                                                    float& power_floor, float& mark_limit) {
  const float4 cp = cull_params(co, power_floor);
  const float far_x = fmaxf(fabsf(xy.x - tile_x0), fabsf(xy.x - (tile_x0 + (float)(GS_TILE_X - 1))));
  const float far_y = fmaxf(fabsf(xy.y - tile_y0), fabsf(xy.y - (tile_y0 + (float)(GS_TILE_Y - 1))));
  const float spread = co.x * far_x * far_x + 2.0f * fabsf(co.y) * far_x * far_y + co.z * far_y * far_y;
  // (q_max = 2 (tau + 0.01) is -2 power_floor wherever the conic is trusted)
  mark_limit = __builtin_fmaf(2e-6f, spread, -2.0f * power_floor);
  const bool never = cp.z < 0.f, untrusted = cp.z == __builtin_inff();
  return make_float4(cp.x, cp.y, never ? -1.0f : (untrusted ? cp.z : mark_limit), 0.f);
}

// The four 4x4 pixel blocks of an 8x8 quadrant at (qx0, qy0), block r at x offset 4 (r & 1), y offset 4 (r >> 1):
// hit[r] = can any point of block r have q <= limit?  q is convex, so over a block it is smallest either at the
// centre (inside the block: 0) or on one of the two block edges that face the centre; along an edge it is a
// parabola whose minimiser is clamped to the edge.  A block is treated as a continuous rectangle, which can only
// add hits.  What the two columns and the two rows of blocks have in common is computed once; the parabolas are
// evaluated in Horner form with fused multiply-adds.  inv_a, inv_c and limit: block_test_params.  NaNs count as
// hits.
__device__ __forceinline__ void ellipse_hits_quadrant(float2 mu, float4 co, float inv_a, float inv_c, float limit,
                                                      float qx0, float qy0, bool (&hit)[4]) {
  const float two_b = 2.0f * co.y;
  float lox[2], hix[2], dxc[2], t1[2], a1[2], b1[2];  // per column of blocks
  float loy[2], hiy[2], dyc[2], t2[2], a2[2], b2[2];  // per row of blocks
#pragma unroll
  for (int c = 0; c < 2; c++) {
    lox[c] = (qx0 + (float)(4 * c)) - mu.x;
    hix[c] = lox[c] + 3.0f;
    dxc[c] = fminf(fmaxf(0.f, lox[c]), hix[c]);  // offset of the nearest column of the block
    t1[c] = -co.y * dxc[c] * inv_c;              // where q is smallest along that column
    a1[c] = co.x * dxc[c] * dxc[c];
    b1[c] = two_b * dxc[c];
    loy[c] = (qy0 + (float)(4 * c)) - mu.y;
    hiy[c] = loy[c] + 3.0f;
    dyc[c] = fminf(fmaxf(0.f, loy[c]), hiy[c]);  // offset of the nearest row of the block
    t2[c] = -co.y * dyc[c] * inv_a;              // where q is smallest along that row
    a2[c] = co.z * dyc[c] * dyc[c];
    b2[c] = two_b * dyc[c];
  }
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int c = r & 1, d = r >> 1;
    const float dy1 = fminf(fmaxf(t1[c], loy[d]), hiy[d]);  // best point of the column x = dxc
    const float q1 = __builtin_fmaf(__builtin_fmaf(co.z, dy1, b1[c]), dy1, a1[c]);
    const float dx2 = fminf(fmaxf(t2[d], lox[c]), hix[c]);  // best point of the row y = dyc
    const float q2 = __builtin_fmaf(__builtin_fmaf(co.x, dx2, b2[d]), dx2, a2[d]);
    hit[r] = !(fminf(q1, q2) > limit);
  }
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

// ---- 4x4-pixel rows -------------------------------------------------------
// Inside a wave's 8x8 quadrant every 16-lane DPP row owns a 4x4 pixel block
// (row r at x offset 4*(r&1), y offset 4*(r>>1); lane l16 of the row is pixel
// (l16 & 3, l16 >> 2) of the block).  The blend loops let the four rows of a
// wave walk four different Gaussians at the same time, each row following its
// own list of Gaussians whose box meets its 4x4 block.
struct RowThread {
  int lane, wave, row, l16;
  uint32_t px, py;
  float qx0, qy0;  // top-left pixel of the wave's quadrant
};

__device__ __forceinline__ RowThread row_thread(uint32_t tile_x, uint32_t tile_y) {
  RowThread t;
  const int tid = threadIdx.x;
  t.lane = tid & (GS_WAVE - 1);
  t.wave = tid / GS_WAVE;
  t.row = t.lane >> 4;
  t.l16 = t.lane & 15;
  const uint32_t x0 = tile_x * GS_TILE_X + (uint32_t)(t.wave & 1) * 8u;
  const uint32_t y0 = tile_y * GS_TILE_Y + (uint32_t)(t.wave >> 1) * 8u;
  t.px = x0 + (uint32_t)(t.row & 1) * 4u + (uint32_t)(t.l16 & 3);
  t.py = y0 + (uint32_t)(t.row >> 1) * 4u + (uint32_t)(t.l16 >> 2);
  t.qx0 = (float)x0;
  t.qy0 = (float)y0;
  return t;
}

template <int CTRL, int BANK_MASK>
__device__ __forceinline__ float dpp_merge(float old, float src) {
  // lanes of the enabled banks read src through the DPP pattern, the others keep old
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src), CTRL, 0xF, BANK_MASK, false));
}

// Transposing reduction inside every 16-lane row: on entry each lane holds 16
// values, on return lane l16 of a row holds the sum over the row's 16 lanes of
// value number l16.  Four halving steps (distances 8, 4, 2, 1): at each step a
// lane keeps half of its values and adds the partner lane's copy of them, so
// 8 + 4 + 2 + 1 lane-pair sums replace 16 x 4.  Written as DPP additions whose
// bank mask selects which lanes of a row take the result, two instructions per
// kept value in the first two steps (33 VALU instructions in all); v[0..7] are
// overwritten.  All 64 lanes must be active.
__device__ __forceinline__ float row_transpose_reduce16(float* v) {
  const uint64_t bit1_lanes = 0xCCCCCCCCCCCCCCCCull, bit0_lanes = 0xAAAAAAAAAAAAAAAAull;
  // A DPP operand written by the preceding VALU instruction needs two idle issue slots first; the s_nop 1
  // between the steps provide them, inside a step no instruction reads a register written less than two
  // instructions earlier through DPP.
  asm volatile(
      "s_nop 1\n\t"
      // distance 8: lanes 0-7 of a row keep values 0-7, lanes 8-15 keep values 8-15
      "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %4, %4, %4 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %5, %5, %5 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %6, %6, %6 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %7, %7, %7 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %4, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %5, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %6, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %7, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "s_nop 1\n\t"
      // distance 4: lanes with bit 2 clear (banks 0, 2) keep registers 0-3 and add lane +4's copy,
      // the others keep registers 4-7 and add lane -4's copy
      "v_add_f32_dpp %0, %0, %0 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %1, %1, %1 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %2, %2, %2 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %3, %3, %3 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %0, %4, %4 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %1, %5, %5 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %2, %6, %6 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %3, %7, %7 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "s_nop 1\n\t"
      // distance 2: + lane^2; lanes with bit 1 set keep registers 2, 3
      "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %2, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, %3, %3 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, %2, %16\n\t"
      "v_cndmask_b32_e64 %1, %1, %3, %16\n\t"
      "s_nop 1\n\t"
      // distance 1: + lane^1; lanes with bit 0 set keep register 1
      "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_cndmask_b32_e64 %0, %0, %1, %17\n\t"
      : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
      : "v"(v[8]), "v"(v[9]), "v"(v[10]), "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]),
        "s"(bit1_lanes), "s"(bit0_lanes));
  return v[0];
}

// The same with values 2 and 3 defined as |value 0| and |value 1|: their first step reads v[0] and v[1] through the
// absolute-value source modifier (before those registers are overwritten), so the caller never forms them; v[2] and
// v[3] need not be set on entry.
__device__ __forceinline__ float row_transpose_reduce16_abs23(float* v) {
  const uint64_t bit1_lanes = 0xCCCCCCCCCCCCCCCCull, bit0_lanes = 0xAAAAAAAAAAAAAAAAull;
  // A DPP operand written by the preceding VALU instruction needs two idle issue slots first; the s_nop 1
  // between the steps provide them, inside a step no instruction reads a register written less than two
  // instructions earlier through DPP.
  asm volatile(
      "s_nop 1\n\t"
      // distance 8: lanes 0-7 of a row keep values 0-7, lanes 8-15 keep values 8-15
      "v_add_f32_dpp %2, |%0|, |%0| row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, |%1|, |%1| row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %4, %4, %4 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %5, %5, %5 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %6, %6, %6 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %7, %7, %7 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %4, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %5, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %6, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "v_add_f32_dpp %7, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "s_nop 1\n\t"
      // distance 4: lanes with bit 2 clear (banks 0, 2) keep registers 0-3 and add lane +4's copy,
      // the others keep registers 4-7 and add lane -4's copy
      "v_add_f32_dpp %0, %0, %0 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %1, %1, %1 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %2, %2, %2 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %3, %3, %3 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %0, %4, %4 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %1, %5, %5 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %2, %6, %6 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %3, %7, %7 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "s_nop 1\n\t"
      // distance 2: + lane^2; lanes with bit 1 set keep registers 2, 3
      "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %2, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, %3, %3 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, %2, %16\n\t"
      "v_cndmask_b32_e64 %1, %1, %3, %16\n\t"
      "s_nop 1\n\t"
      // distance 1: + lane^1; lanes with bit 0 set keep register 1
      "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_cndmask_b32_e64 %0, %0, %1, %17\n\t"
      : "+v"(v[0]), "+v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
      : "v"(v[8]), "v"(v[9]), "v"(v[10]), "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]),
        "s"(bit1_lanes), "s"(bit0_lanes));
  return v[0];
}

}  // namespace gs

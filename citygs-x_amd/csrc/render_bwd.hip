// Backward of the per-tile blend (cuda_rasterizer/backward.cu:324-567): each
// pixel replays its Gaussians back to front from the stored final
// transmittance and contributor count, and per-Gaussian gradients are summed
// over pixels.
//
// Workgroup = one 16x16 tile = four 64-lane waves.  All lanes of a wave visit
// the same Gaussian at the same time, so the 17 per-Gaussian partial sums are
// first reduced across the wave with DPP row operations (quad swaps, row
// rotations, row broadcasts: no LDS traffic), and only lane 63 issues the
// global float atomics: one atomic per wave and component instead of one per
// pixel.  Waves in which no lane touches the Gaussian skip the reduction.
// Summation order therefore differs from a per-pixel atomic order; gradients
// agree with a CPU evaluation to rounding, not bit for bit.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int BATCH = GS_TILE_PIX;

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
  return v + __int_as_float(moved);
}

// Sum over the 64 lanes; the total is valid in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x124, 0xF>(v);  // row_ror:4
  v = dpp_add<0x128, 0xF>(v);  // row_ror:8  -> every lane holds its row's sum
  v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

__global__ void __launch_bounds__(GS_TILE_PIX)
render_bwd_kernel(const uint2* __restrict__ ranges, const uint32_t* __restrict__ point_list, int W, int H, float fx,
                  float fy, const float* __restrict__ bg, const float2* __restrict__ means2D,
                  const float4* __restrict__ conic_opacity, const float* __restrict__ rgb,
                  const float* __restrict__ all_map, const float* __restrict__ all_map_pixels,
                  const float* __restrict__ final_Ts, const uint32_t* __restrict__ n_contrib_px,
                  const uint8_t* __restrict__ compute_locally, const float* __restrict__ dL_dpix,
                  const float* __restrict__ dL_dout_all_map, const float* __restrict__ dL_dout_plane_depth,
                  int render_geo, float* __restrict__ dL_dmean2D, float* __restrict__ dL_dmean2D_abs,
                  float* __restrict__ dL_dconic_opacity, float* __restrict__ dL_dcolors,
                  float* __restrict__ dL_dall_map) {
  __shared__ int s_id[BATCH];
  __shared__ float2 s_xy[BATCH];
  __shared__ float4 s_co[BATCH];
  __shared__ float s_rgb[GS_N_RGB][BATCH];
  __shared__ float s_map[GS_N_MAP][BATCH];

  const int tid = threadIdx.y * GS_TILE_X + threadIdx.x;
  const int lane = tid & (GS_WAVE - 1);
  const uint32_t tile = blockIdx.y * gridDim.x + blockIdx.x;
  if (!compute_locally[tile]) return;
  const uint32_t px = blockIdx.x * GS_TILE_X + threadIdx.x, py = blockIdx.y * GS_TILE_Y + threadIdx.y;
  const bool inside = px < (uint32_t)W && py < (uint32_t)H;
  const size_t pid = (size_t)W * py + px;
  const size_t HW = (size_t)H * W;
  const float pfx = (float)px, pfy = (float)py;
  const float rayx = (float)(((double)pfx - W * 0.5) / (double)fx);
  const float rayy = (float)(((double)pfy - H * 0.5) / (double)fy);
  const uint2 range = ranges[tile];
  int todo = (int)(range.y - range.x);
  const int rounds = (todo + BATCH - 1) / BATCH;

  const float T_final = inside ? final_Ts[pid] : 0.f;
  float T = T_final;
  uint32_t contributor = (uint32_t)todo;
  const int last_contributor = inside ? (int)n_contrib_px[pid] : 0;

  float accum_rec[GS_N_RGB] = {0.f, 0.f, 0.f}, accum_map[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
  float gpix[GS_N_RGB] = {0.f, 0.f, 0.f}, gmap[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
  if (inside) {
#pragma unroll
    for (int ch = 0; ch < GS_N_RGB; ch++) gpix[ch] = dL_dpix[ch * HW + pid];
    if (render_geo) {
#pragma unroll
      for (int ch = 0; ch < GS_N_MAP; ch++) gmap[ch] = dL_dout_all_map[ch * HW + pid];
      const float nx = all_map_pixels[pid], ny = all_map_pixels[HW + pid], nz = all_map_pixels[2 * HW + pid];
      const float dist = all_map_pixels[4 * HW + pid];
      const float tmp = (float)((double)((nx * rayx + ny * rayy) + nz) + 1.0e-8);
      const float gd = dL_dout_plane_depth[pid];
      gmap[GS_N_MAP - 1] += (-gd / tmp);
      gmap[0] += gd * (dist / (tmp * tmp) * rayx);
      gmap[1] += gd * (dist / (tmp * tmp) * rayy);
      gmap[2] += gd * (dist / (tmp * tmp));
    }
  }
  float bg_dot = 0.f;
#pragma unroll
  for (int ch = 0; ch < GS_N_RGB; ch++) bg_dot += bg[ch] * gpix[ch];

  float last_alpha = 0.f;
  float last_color[GS_N_RGB] = {0.f, 0.f, 0.f}, last_map[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};
  const float ddelx_dx = (float)(0.5 * W), ddely_dy = (float)(0.5 * H);

  for (int i = 0; i < rounds; i++, todo -= BATCH) {
    __syncthreads();
    const uint32_t progress = (uint32_t)i * BATCH + tid;
    if (range.x + progress < range.y) {
      const uint32_t g = point_list[range.y - progress - 1];
      s_id[tid] = (int)g;
      s_xy[tid] = means2D[g];
      s_co[tid] = conic_opacity[g];
      s_rgb[0][tid] = rgb[3 * (size_t)g];
      s_rgb[1][tid] = rgb[3 * (size_t)g + 1];
      s_rgb[2][tid] = rgb[3 * (size_t)g + 2];
      if (render_geo) {
#pragma unroll
        for (int ch = 0; ch < GS_N_MAP; ch++) s_map[ch][tid] = all_map[5 * (size_t)g + ch];
      }
    }
    __syncthreads();

    const int count = todo < BATCH ? todo : BATCH;
    for (int j = 0; j < count; j++) {
      contributor--;
      bool active = inside && ((int)contributor < last_contributor);
      float dx = 0.f, dy = 0.f, G = 0.f, alpha = 0.f;
      float4 co = make_float4(0.f, 0.f, 0.f, 0.f);
      if (active) {
        const float2 xy = s_xy[j];
        dx = xy.x - pfx;
        dy = xy.y - pfy;
        co = s_co[j];
        const float power = -0.5f * (co.x * dx * dx + co.z * dy * dy) - co.y * dx * dy;
        if (power > 0.0f) {
          active = false;
        } else {
          G = gs_expf(power);
          alpha = fminf(0.99f, co.w * G);
          if (alpha < 1.0f / 255.0f) active = false;
        }
      }
      if (__ballot(active) == 0ull) continue;  // wave-uniform

      float v[17];
#pragma unroll
      for (int q = 0; q < 17; q++) v[q] = 0.f;
      if (active) {
        T = T / (1.f - alpha);
        const float w = alpha * T;
        float dL_dalpha = 0.0f;
#pragma unroll
        for (int ch = 0; ch < GS_N_RGB; ch++) {
          const float c = s_rgb[ch][j];
          accum_rec[ch] = last_alpha * last_color[ch] + (1.f - last_alpha) * accum_rec[ch];
          last_color[ch] = c;
          dL_dalpha += (c - accum_rec[ch]) * gpix[ch];
          v[9 + ch] = w * gpix[ch];
        }
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) {
            const float c = s_map[ch][j];
            accum_map[ch] = last_alpha * last_map[ch] + (1.f - last_alpha) * accum_map[ch];
            last_map[ch] = c;
            dL_dalpha += (c - accum_map[ch]) * gmap[ch];
            v[12 + ch] = w * gmap[ch];
          }
        }
        dL_dalpha *= T;
        last_alpha = alpha;
        dL_dalpha += (-T_final / (1.f - alpha)) * bg_dot;
        const float dL_dG = co.w * dL_dalpha;
        const float gdx = G * dx, gdy = G * dy;
        const float dG_ddelx = -gdx * co.x - gdy * co.y;
        const float dG_ddely = -gdy * co.z - gdx * co.y;
        v[0] = dL_dG * dG_ddelx * ddelx_dx;
        v[1] = dL_dG * dG_ddely * ddely_dy;
        v[2] = fabsf(v[0]);
        v[3] = fabsf(v[1]);
        v[4] = -0.5f * gdx * dx * dL_dG;
        v[5] = -0.5f * gdx * dy * dL_dG;
        v[6] = -0.5f * gdy * dy * dL_dG;
        v[7] = G * dL_dalpha;
      }
      const int nred = render_geo ? 17 : 12;
#pragma unroll
      for (int q = 0; q < 17; q++)
        if (q != 8 && q < nred) v[q] = wave_sum_to_lane63(v[q]);
      if (lane == GS_WAVE - 1) {
        const size_t g = (size_t)s_id[j];
        unsafeAtomicAdd(&dL_dmean2D[2 * g], v[0]);
        unsafeAtomicAdd(&dL_dmean2D[2 * g + 1], v[1]);
        unsafeAtomicAdd(&dL_dmean2D_abs[3 * g], v[2]);
        unsafeAtomicAdd(&dL_dmean2D_abs[3 * g + 1], v[3]);
        unsafeAtomicAdd(&dL_dconic_opacity[4 * g], v[4]);
        unsafeAtomicAdd(&dL_dconic_opacity[4 * g + 1], v[5]);
        unsafeAtomicAdd(&dL_dconic_opacity[4 * g + 2], v[6]);
        unsafeAtomicAdd(&dL_dconic_opacity[4 * g + 3], v[7]);
#pragma unroll
        for (int ch = 0; ch < GS_N_RGB; ch++) unsafeAtomicAdd(&dL_dcolors[3 * g + ch], v[9 + ch]);
        if (render_geo) {
#pragma unroll
          for (int ch = 0; ch < GS_N_MAP; ch++) unsafeAtomicAdd(&dL_dall_map[5 * g + ch], v[12 + ch]);
        }
      }
    }
  }
}

}  // namespace

int launch_render_bwd(const RenderBwdArgs& a, hipStream_t stream) {
  const dim3 grid((a.W + GS_TILE_X - 1) / GS_TILE_X, (a.H + GS_TILE_Y - 1) / GS_TILE_Y, 1);
  const dim3 block(GS_TILE_X, GS_TILE_Y, 1);
  hipLaunchKernelGGL(render_bwd_kernel, grid, block, 0, stream, (const uint2*)a.ranges, a.point_list, a.W, a.H, a.fx,
                     a.fy, a.bg, (const float2*)a.means2D, (const float4*)a.conic_opacity, a.rgb, a.all_map,
                     a.all_map_pixels, a.final_T, a.n_contrib_px, a.compute_locally, a.dL_dpix, a.dL_dout_all_map,
                     a.dL_dout_plane_depth, a.render_geo, a.dL_dmean2D, a.dL_dmean2D_abs, a.dL_dconic_opacity,
                     a.dL_dcolors, a.dL_dall_map);
  return 0;
}

}  // namespace gs

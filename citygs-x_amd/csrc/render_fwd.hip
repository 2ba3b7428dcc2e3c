// Per-tile front-to-back alpha blending (cuda_rasterizer/forward.cu:264-437)
// with the per-tile statistics of cuda_rasterizer/rasterizer_impl.cu:219-262
// folded into the same kernel.
//
// One 256-thread workgroup per 16x16 tile; each of its four 64-lane waves owns
// an 8x8 pixel quadrant.  The tile's depth-sorted Gaussians are staged through
// LDS in batches of 256 (index, centre, conic+opacity, colour, the five
// geometry channels, and a conservative screen-space box).  Per batch every
// wave builds four 64-bit ballots of the Gaussians whose box meets its
// quadrant and then walks only the set bits with scalar bit scans, so a
// Gaussian that cannot touch the quadrant costs the wave nothing.  A wave
// leaves the walk as soon as all its pixels have saturated, and a batch is
// not even fetched once all four waves have.
//
// The per-pixel arithmetic keeps the operation order of the reference, so
// contributor counts (and in practice the images) match a CPU evaluation bit
// for bit; exp() is gs_expf.  out_observe increments are summed per wave with
// a ballot and per workgroup in LDS, then added once per (tile, Gaussian).
#include "gs_common.h"
#include "gs_kernels.h"
#include "render_common.h"

namespace gs {

namespace {

constexpr int BATCH = GS_TILE_PIX;

__global__ void __launch_bounds__(GS_TILE_PIX)
render_fwd_kernel(const uint2* __restrict__ ranges, const uint32_t* __restrict__ point_list, int W, int H, float fx,
                  float fy, float cx, float cy, const float2* __restrict__ means2D, const float* __restrict__ rgb,
                  const float* __restrict__ all_map, const float4* __restrict__ conic_opacity,
                  const uint8_t* __restrict__ compute_locally, const float* __restrict__ bg, int render_geo,
                  float* __restrict__ final_T, uint32_t* __restrict__ n_contrib_px,
                  uint32_t* __restrict__ n_contrib2loss_px, float* __restrict__ out_color,
                  int* __restrict__ out_observe, float* __restrict__ out_all_map,
                  float* __restrict__ out_plane_depth, int* __restrict__ n_render, int* __restrict__ n_consider,
                  int* __restrict__ n_contrib_tile) {
  __shared__ int s_id[BATCH];
  __shared__ float2 s_xy[BATCH];
  __shared__ float4 s_co[BATCH];
  __shared__ float4 s_bb[BATCH];
  __shared__ float s_floor[BATCH];
  __shared__ float s_rgb[GS_N_RGB][BATCH];
  __shared__ float s_map[GS_N_MAP][BATCH];
  __shared__ int s_obs[BATCH];
  __shared__ int s_done[GS_TILE_PIX / GS_WAVE];
  __shared__ int s_red[2][GS_TILE_PIX / GS_WAVE];

  const int tid = threadIdx.x;
  const TileThread tt = tile_thread(blockIdx.x, blockIdx.y);
  const int lane = tt.lane, wave = tt.wave;
  const uint32_t tile = blockIdx.y * gridDim.x + blockIdx.x;
  const uint2 range = ranges[tile];
  if (tid == 0) n_render[tile] = (int)(range.y - range.x);
  if (!compute_locally[tile]) {
    if (tid == 0) {
      n_consider[tile] = 0;
      n_contrib_tile[tile] = 0;
    }
    return;
  }
  const uint32_t px = tt.px, py = tt.py;
  const bool inside = px < (uint32_t)W && py < (uint32_t)H;
  const size_t pid = (size_t)W * py + px;
  const float pfx = (float)px, pfy = (float)py;
  const float rayx = (pfx - cx) / fx, rayy = (pfy - cy) / fy;
  bool done = !inside;

  int todo = (int)(range.y - range.x);
  const int rounds = (todo + BATCH - 1) / BATCH;

  float T = 1.0f;
  uint32_t last = 0, n2l = 0;
  float C[GS_N_RGB] = {0.f, 0.f, 0.f};
  float Mp[GS_N_MAP] = {0.f, 0.f, 0.f, 0.f, 0.f};

  for (int i = 0; i < rounds; i++, todo -= BATCH) {
    const bool wave_done = __ballot(!done) == 0ull;
    if (lane == 0) s_done[wave] = wave_done;
    __syncthreads();
    if (s_done[0] && s_done[1] && s_done[2] && s_done[3]) break;

    const int count = todo < BATCH ? todo : BATCH;
    if (tid < count) {
      const uint32_t g = point_list[range.x + (uint32_t)i * BATCH + tid];
      const float2 xy = means2D[g];
      const float4 co = conic_opacity[g];
      s_id[tid] = (int)g;
      s_xy[tid] = xy;
      s_co[tid] = co;
      float pfl;
      s_bb[tid] = cull_box(xy, co, pfl);
      s_floor[tid] = pfl;
      s_rgb[0][tid] = rgb[3 * (size_t)g];
      s_rgb[1][tid] = rgb[3 * (size_t)g + 1];
      s_rgb[2][tid] = rgb[3 * (size_t)g + 2];
      if (render_geo) {
#pragma unroll
        for (int ch = 0; ch < GS_N_MAP; ch++) s_map[ch][tid] = all_map[5 * (size_t)g + ch];
      }
    }
    s_obs[tid] = 0;
    __syncthreads();

    if (!wave_done) {
      // which Gaussians of the batch can touch this wave's 8x8 quadrant
      uint64_t rel[BATCH / GS_WAVE];
#pragma unroll
      for (int k = 0; k < BATCH / GS_WAVE; k++) {
        const int j = k * GS_WAVE + lane;
        rel[k] = __ballot(j < count && box_hits_wave(s_bb[j], tt));
      }
      bool alive = true;
#pragma unroll
      for (int k = 0; k < BATCH / GS_WAVE; k++) {
        uint64_t m = alive ? rel[k] : 0ull;
        while (m != 0ull) {
          const int j = k * GS_WAVE + (int)__builtin_ctzll(m);
          m &= m - 1ull;
          // exponent first; the exponential only for lanes that can still pass the 1/255 test
          float power = 0.f, o = 0.f;
          bool in = false;
          if (!done) {
            const float2 xy = s_xy[j];
            const float dx = xy.x - pfx, dy = xy.y - pfy;
            const float4 co = s_co[j];
            o = co.w;
            power = -0.5f * (co.x * dx * dx + co.z * dy * dy) - co.y * dx * dy;
            in = !(power > 0.0f) && !(power < s_floor[j]);
          }
          if (__ballot(in) == 0ull) continue;
          bool blend = false;
          float alpha = 0.f, test_T = 0.f;
          if (in) {
            alpha = fminf(0.99f, o * gs_expf_core(power));
            if (!(alpha < 1.0f / 255.0f)) {
              test_T = T * (1 - alpha);
              if (test_T < 0.0001f)
                done = true;
              else
                blend = true;
            }
          }
          const uint64_t bmask = __ballot(blend);
          if (bmask != 0ull) {
            if (blend) {
              n2l++;
              // weight once, then one fused multiply-add per channel (image values are held to 1e-4, not to the bit)
              const float w = alpha * T;
#pragma unroll
              for (int ch = 0; ch < GS_N_RGB; ch++) C[ch] = __builtin_fmaf(s_rgb[ch][j], w, C[ch]);
              if (render_geo) {
#pragma unroll
                for (int ch = 0; ch < GS_N_MAP; ch++) Mp[ch] = __builtin_fmaf(s_map[ch][j], w, Mp[ch]);
              }
            }
            const uint64_t omask = __ballot(blend && T > 0.5f);
            if (omask != 0ull && lane == 0) atomicAdd(&s_obs[j], (int)__popcll(omask));
            if (blend) {
              T = test_T;
              last = (uint32_t)(i * BATCH + j + 1);
            }
          }
          if (__ballot(!done) == 0ull) {
            m = 0ull;
            alive = false;  // every pixel of this wave has saturated
          }
        }
      }
    }
    __syncthreads();
    if (tid < count) {
      const int c = s_obs[tid];
      if (c != 0) atomicAdd(&out_observe[s_id[tid]], c);
    }
  }

  if (inside) {
    const size_t HW = (size_t)H * W;
    final_T[pid] = T;
    n_contrib_px[pid] = last;
    n_contrib2loss_px[pid] = n2l;
#pragma unroll
    for (int ch = 0; ch < GS_N_RGB; ch++) out_color[ch * HW + pid] = C[ch] + T * bg[ch];
    if (render_geo) {
#pragma unroll
      for (int ch = 0; ch < GS_N_MAP; ch++) out_all_map[ch * HW + pid] = Mp[ch];
      const float den_f = (Mp[0] * rayx + Mp[1] * rayy) + Mp[2];
      out_plane_depth[pid] = (float)((double)Mp[4] / -((double)den_f + 1.0e-8));
    }
  }

  // per-tile integer sums of the two per-pixel counters
  int a = inside ? (int)last : 0, b = inside ? (int)n2l : 0;
#pragma unroll
  for (int d = GS_WAVE / 2; d >= 1; d >>= 1) {
    a += __shfl_xor(a, d, GS_WAVE);
    b += __shfl_xor(b, d, GS_WAVE);
  }
  __syncthreads();
  if (lane == 0) {
    s_red[0][wave] = a;
    s_red[1][wave] = b;
  }
  __syncthreads();
  if (tid == 0) {
    n_consider[tile] = s_red[0][0] + s_red[0][1] + s_red[0][2] + s_red[0][3];
    n_contrib_tile[tile] = s_red[1][0] + s_red[1][1] + s_red[1][2] + s_red[1][3];
  }
}

}  // namespace

int launch_render_fwd(const RenderFwdArgs& a, hipStream_t stream) {
  const dim3 grid((a.W + GS_TILE_X - 1) / GS_TILE_X, (a.H + GS_TILE_Y - 1) / GS_TILE_Y, 1);
  hipLaunchKernelGGL(render_fwd_kernel, grid, dim3(GS_TILE_PIX), 0, stream, (const uint2*)a.ranges, a.point_list, a.W,
                     a.H, a.fx, a.fy, a.cx, a.cy, (const float2*)a.means2D, a.rgb, a.all_map,
                     (const float4*)a.conic_opacity, a.compute_locally, a.bg, a.render_geo, a.final_T, a.n_contrib_px,
                     a.n_contrib2loss_px, a.out_color, a.out_observe, a.out_all_map, a.out_plane_depth, a.n_render,
                     a.n_consider, a.n_contrib_tile);
  return 0;
}

}  // namespace gs
